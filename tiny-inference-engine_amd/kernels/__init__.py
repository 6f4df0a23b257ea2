"""The operations of the engine, each one a hand-written HIP kernel for gfx950.

Every function here checks its operands on the host (device, dtype, shape,
contiguity) and then launches the kernel on the current HIP stream. There is
no CPU path: an operand that is not on a GPU, a missing compiler or a library
that cannot be loaded raise KernelUnavailable. Sizes a kernel cannot take raise
InvalidArgument before anything is launched.
"""

from __future__ import annotations

import ctypes
import functools
from typing import Dict, Optional

import torch

from ..errors import InvalidArgument, KernelUnavailable
from . import build

F32, BF16, F16 = 0, 1, 2
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
_CACHE_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}

# The cache of keys and values has a precision of its own (the reference's KVCacheConfig.dtype,
# src/kv/paged_kv_cache.h:18-25: float32 arithmetic over a narrower cache is its default arrangement). Per
# compute mode, the cache dtypes some kernel here reads and writes; the first is the mode's default.
CACHE_DTYPES = {"float32": ("float32", "bfloat16", "float16"), "bfloat16": ("bfloat16",)}
_CACHE_DTYPE_NAMES = {"float32": "float32", "fp32": "float32", "f32": "float32", "bfloat16": "bfloat16",
                      "bf16": "bfloat16", "float16": "float16", "fp16": "float16", "f16": "float16"}


def cache_dtype_for(mode: str, asked: Optional[str] = None) -> str:
    """The cache dtype a compute mode runs over: its own by default, ``asked`` if the kernels take the pair."""
    if mode not in CACHE_DTYPES:
        raise InvalidArgument(f"unknown compute mode '{mode}'")
    if asked is None:
        return CACHE_DTYPES[mode][0]
    name = _CACHE_DTYPE_NAMES.get(asked)
    if name is None:
        raise InvalidArgument(f"the cache dtype must be float32, bfloat16 or float16, got '{asked}'")
    if name not in CACHE_DTYPES[mode]:
        raise InvalidArgument(f"no kernel runs {mode} arithmetic over a {name} cache: with --dtype {mode} the cache "
                              f"can be {' or '.join(CACHE_DTYPES[mode])} (the matrix-core attention kernels read "
                              f"bfloat16 pages; float32 arithmetic reads any of the three)")
    return name

_c_int, _c_float, _c_void, _c_long = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_long

# library key -> (file stem, source)
_SOURCES = {
    "elementwise": ("tie_elementwise", "elementwise.hip"),
    "gemm_generic": ("tie_gemm_generic", "gemm_generic.hip"),
    "attention_generic": ("tie_attention_generic", "attention_generic.hip"),
    "skinny_gemm_bf16": ("tie_skinny_gemm_bf16", "skinny_gemm_bf16.hip"),
    "gemm_bf16": ("tie_gemm_bf16", "gemm_bf16.hip"),
    "sample_filtered": ("tie_sample_filtered", "sample_filtered.hip"),
    "machine_peaks": ("tie_machine_peaks", "machine_peaks.hip"),
    "moe": ("tie_moe", "moe.hip"),
    "recurrent": ("tie_recurrent", "recurrent.hip"),
    "hyper": ("tie_hyper", "hyper.hip"),
    "delta_rule": ("tie_delta_rule", "delta_rule.hip"),
    "latent": ("tie_latent", "latent.hip"),
    "pointwise": ("tie_pointwise", "pointwise.hip"),
}
# libraries compiled once per head size: key -> (file stem prefix, source)
_PER_HEAD_DIM = {
    "attention_decode_bf16": ("tie_attention_decode_bf16", "attention_decode_bf16.hip"),
    "attention_prefill_bf16": ("tie_attention_prefill_bf16", "attention_prefill_bf16.hip"),
}
MFMA_HEAD_DIMS = tuple(range(16, 257, 16))   # head sizes the matrix-core attention kernels are built for
MAX_KEY_SPLITS = 256      # MERGE_MAX_SPLITS of csrc/attention_merge.h: the most shares one row's keys are cut into
MAX_HEAD_DIM = 512        # the largest head size any attention kernel takes (the generic ones)
MAX_STEP_TOKENS = 65535   # rows of one step: a grid dimension of the row-wise kernels

_SIGNATURES = {
    "machine_peaks": {
        "tie_stream_read": [_c_void, ctypes.c_longlong, _c_int, _c_void, _c_void, _c_void],
        "tie_mfma_rate": [_c_int, _c_int, _c_void, _c_void, _c_void],
    },
    "sample_filtered": {
        "tie_sample_filtered": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                _c_int, _c_void, _c_int, _c_int, _c_void],
    },
    "elementwise": {
        "tie_embed": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_int, _c_float, _c_void],
        "tie_poly_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_scale_softcap": [_c_void, ctypes.c_longlong, _c_float, _c_float, _c_void],
        "tie_rms_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
        "tie_swiglu": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void],
        "tie_cast": [_c_void, _c_int, _c_void, _c_int, ctypes.c_longlong, _c_void],
        "tie_scale_rows": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_int, _c_float, _c_float, _c_void],
        "tie_add_bias": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_take_tokens": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_random_fill": [_c_void, ctypes.c_longlong, ctypes.c_ulonglong, _c_int, ctypes.c_double, _c_void],
        "tie_rope_angles": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_float, _c_void],
        "tie_qk_norm_rope_kv_write": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_float, _c_void, _c_void,
                                      _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_long, _c_int, _c_int, _c_int,
                                      _c_void, _c_void, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_norm_add_norm": [_c_void, _c_long, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void,
                              _c_float, _c_void, _c_void, _c_float, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_gelu": [_c_void, _c_int, _c_void, _c_int, ctypes.c_longlong, _c_void],
        "tie_add_partials_rms_norm": [_c_void, _c_void, _c_long, _c_int, _c_void, _c_float, _c_void, _c_int, _c_int,
                                      _c_int, _c_void],
        "tie_argmax": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_sample": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_void, _c_int,
                       _c_int, _c_void],
        "tie_argmax_static": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
    },
    "moe": {
        "tie_moe_route": [_c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_float, _c_float, _c_int, _c_void, _c_void, _c_void],
        "tie_moe_max_tiles": [_c_int, _c_int, _c_int],
        "tie_moe_align": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void],
        "tie_moe_generic_tile_rows": [],
        "tie_moe_gemm_generic": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void, _c_void,
                                 _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void],
        "tie_moe_bf16_tile_rows": [_c_int, _c_int],
        "tie_moe_gemm_bf16": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int,
                              _c_int, _c_int, _c_int, _c_int, _c_void],
        "tie_moe_combine": [_c_void, _c_void, _c_void, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void],
    },
    "gemm_generic": {
        "tie_gemm_generic": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int,
                             _c_void],
    },
    "attention_generic": {
        "tie_paged_attention_generic": [_c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void, _c_void,
                                        _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                        _c_float, _c_int, _c_int, _c_int, _c_void, _c_void],
    },
    "recurrent": {
        "tie_decay_attention_scan": [_c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int,
                                     _c_int, _c_int, _c_int, _c_void, _c_void, _c_int, _c_void, _c_int, _c_void],
        "tie_gated_rms_norm": [_c_void, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_min_gru_scan": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void,
                             _c_void, _c_int, _c_void, _c_void, _c_void],
    },
    "hyper": {
        "tie_layer_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int, _c_void],
        "tie_hyper_connection": [_c_void, _c_long, _c_int, _c_int, _c_void, _c_int, _c_void, _c_long, _c_int, _c_void,
                                 _c_void, _c_void, _c_void, _c_float, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void],
    },
    "delta_rule": {
        "tie_conv_qkv": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int,
                         _c_int, _c_void, _c_void, _c_float, _c_float, _c_float, _c_void, _c_int, _c_void],
        "tie_conv_state_update": [_c_void, _c_int, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_void],
        "tie_delta_prepare": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int,
                              _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void, _c_int, _c_void],
        "tie_gated_delta_scan": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int,
                                 _c_int, _c_int, _c_void],
        "tie_gated_delta_scan_chunked": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_void, _c_int, _c_void, _c_void,
                                         _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_void],
        "tie_grouped_gated_rms_norm": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_void, _c_int, _c_int,
                                       _c_int, _c_int, _c_void],
    },
    "pointwise": {
        "tie_dynamic_tanh": [_c_void, _c_void, _c_long, _c_int, _c_void, _c_void, _c_void, _c_void, _c_int, _c_void,
                             _c_int, _c_int, _c_int, _c_void],
        "tie_token_gate": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void],
    },
    "latent": {
        "tie_rms_norm_columns": [_c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_int, _c_int, _c_void],
        "tie_latent_prepare": [_c_void, _c_int, _c_void, _c_int, _c_void, _c_float, _c_void, _c_int, _c_int, _c_void, _c_void, _c_void,
                               _c_int, _c_int, _c_int, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                               _c_int, _c_void],
        "tie_head_linear": [_c_void, _c_int, _c_int, _c_int, _c_void, _c_int, _c_void, _c_int, _c_int, _c_int, _c_void,
                            _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_void],
    },
    "skinny_gemm_bf16": {
        "tie_skinny_gemm_splits": [_c_int, _c_int],
        "tie_skinny_few_rows_plan": [_c_int, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_skinny_gemm_bf16_with": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                      _c_int, _c_int, _c_int, _c_void],
        "tie_skinny_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_void],
        "tie_skinny_norm_epilogue_rows": [_c_int, _c_int],
        "tie_skinny_gemm_bf16_norm": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                      _c_int, _c_void, _c_int, _c_float, _c_float, _c_void, _c_void, _c_void, _c_int,
                                      _c_int, _c_int, _c_void],
    },
    "gemm_bf16": {
        "tie_gemm_bf16_splits": [_c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16_tile": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16_wins_few_rows": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "tie_gemm_bf16": [_c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_int, _c_void],
    },
    "attention_prefill_bf16": {
        "tie_attention_prefill_rows_per_item": [_c_int],
        "tie_attention_prefill_bf16": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_int,
                                       _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int, _c_int, _c_void, _c_void,
                                       _c_void, _c_int, _c_void],
        "tie_attention_prefill_bf16_with": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                            _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int, _c_int,
                                            _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_void, _c_void],
        "tie_attention_prefill_bf16_keeping": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                               _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int,
                                               _c_int, _c_void, _c_void, _c_void, _c_int, _c_int, _c_int, _c_void,
                                               _c_int, _c_void],
    },
    "attention_decode_bf16": {
        "tie_attention_decode_head_dim": [],
        "tie_attention_max_splits": [],
        "tie_attention_decode_bf16": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                      _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_int, _c_int,
                                      _c_void],
        "tie_attention_decode_prepares": [_c_int],
        "tie_attention_decode_prepared_bf16": [_c_void, _c_long, _c_int, _c_int, _c_void, _c_void, _c_float, _c_void,
                                               _c_int, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                               _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                               _c_int, _c_int, _c_void, _c_int, _c_void],
        "tie_attention_decode_bf16_with": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                           _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float,
                                           _c_int, _c_int, _c_void, _c_int, _c_int, _c_void, _c_void],
        "tie_attention_decode_bf16_keeping": [_c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void, _c_void,
                                              _c_void, _c_void, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                              _c_float, _c_int, _c_int, _c_void, _c_int, _c_int, _c_void, _c_int,
                                              _c_void],
    },
}

_libs = {}


def library_list(head_dims=(16, 32, 48, 64, 80, 96, 112, 128, 256)):
    """``(name, source, defines)`` of every library, for building them all up front.

    The per-head-size libraries are listed for ``head_dims``; any other head size is compiled the
    first time a model with it runs.
    """
    libs = [(stem, source, {}) for stem, source in _SOURCES.values()]
    for stem, source in _PER_HEAD_DIM.values():
        for d in head_dims:
            libs.append((f"{stem}_hd{d}", source, {"HEAD_DIM": d}))
    return libs


def _lib(key: str, head_dim: int = 0):
    cache_key = (key, head_dim)
    lib = _libs.get(cache_key)
    if lib is None:
        if head_dim:
            stem, source = _PER_HEAD_DIM[key]
            lib = build.load_library(f"{stem}_hd{head_dim}", source, {"HEAD_DIM": head_dim})
        else:
            stem, source = _SOURCES[key]
            lib = build.load_library(stem, source)
        for fn, argtypes in _SIGNATURES[key].items():
            f = getattr(lib, fn)
            f.argtypes = argtypes
            f.restype = _c_int
        _libs[cache_key] = lib
    return lib


# The current stream's handle, asked for at every launch. torch's public way (a Stream object built anew each time)
# costs several microseconds a call, which at a few hundred launches a step is milliseconds of a prefill step
# that the GPU then waits for; the raw call behind it costs a fraction of one.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


_recording: Optional[list] = None     # while a list: every launch is also noted in it, as (function, arguments, name)


def start_recording() -> list:
    """From now on every kernel launch is also noted, as ``(function, arguments, name)``; returns the list."""
    global _recording
    _recording = []
    return _recording


def stop_recording() -> None:
    global _recording
    _recording = None


def _call(fn, what: str, *args) -> None:
    """One kernel launch through the C interface: its status checked, the call noted if launches are being recorded."""
    status = fn(*args)
    if _recording is not None:
        _recording.append((fn, args, what))
    _check(status, what)


def replay_call(fn, what: str, args) -> None:
    """A noted launch again, with the arguments given (see ``models.builder``: layers of one shape)."""
    _check(fn(*args), what)


def _check(status: int, what: str) -> None:
    if status == 0:
        return
    if status < 0:
        raise InvalidArgument(f"{what}: the kernel refused its arguments")
    raise KernelUnavailable(f"{what}: HIP error {status} at launch")


def _gpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise InvalidArgument(f"{name} must be a tensor")
    if not t.is_cuda:
        raise KernelUnavailable(
            f"{name} is on '{t.device}': the engine's kernels run on a GPU only and have no CPU fallback")
    if not t.is_contiguous():
        raise InvalidArgument(f"{name} must be contiguous")
    return t


def _gpu_strided(t: torch.Tensor, name: str) -> torch.Tensor:
    """A 2-D GPU tensor whose rows are contiguous but may lie further apart than their width."""
    if not isinstance(t, torch.Tensor) or t.dim() != 2:
        raise InvalidArgument(f"{name} must be a 2-D tensor")
    if not t.is_cuda:
        raise KernelUnavailable(
            f"{name} is on '{t.device}': the engine's kernels run on a GPU only and have no CPU fallback")
    if t.stride(1) != 1 or t.stride(0) < t.shape[1]:
        raise InvalidArgument(f"{name} must have contiguous rows")
    return t


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, KVH: int, block_size: int, Dh: int) -> None:
    """Keys ``[pages, kv heads, block_size, head_dim]``; values transposed in the page ``[pages, kv heads, head_dim, block_size]``."""
    if k_cache.dim() != 4 or v_cache.dim() != 4 or k_cache.dtype != v_cache.dtype or \
            tuple(k_cache.shape[1:]) != (KVH, block_size, Dh) or \
            tuple(v_cache.shape) != (k_cache.shape[0], KVH, Dh, block_size):
        raise InvalidArgument(f"KV cache planes {list(k_cache.shape)} / {list(v_cache.shape)} do not fit "
                              f"{KVH} kv heads, block size {block_size}, head_dim {Dh} "
                              f"(keys [pages, heads, block, dim], values [pages, heads, dim, block])")


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise InvalidArgument(f"{name} must be float32 or bfloat16, got {t.dtype}") from None


def _cache_code(cache: torch.Tensor, beside: torch.Tensor, name: str) -> int:
    """The type code of a cache plane; float16 pages go with float32 activations only."""
    try:
        code = _CACHE_CODES[cache.dtype]
    except KeyError:
        raise InvalidArgument(f"{name} must be float32, bfloat16 or float16, got {cache.dtype}") from None
    if code == F16 and beside.dtype != torch.float32:
        raise InvalidArgument(f"a float16 {name} goes with float32 queries, not {beside.dtype}")
    return code


def _i32(t: torch.Tensor, name: str, numel: Optional[int] = None) -> torch.Tensor:
    _gpu(t, name)
    if t.dtype != torch.int32:
        raise InvalidArgument(f"{name} must be int32, got {t.dtype}")
    if numel is not None and t.numel() < numel:
        raise InvalidArgument(f"{name} holds {t.numel()} entries, {numel} are needed")
    return t


def _f32(t: torch.Tensor, name: str, shape=None) -> torch.Tensor:
    _gpu(t, name)
    if t.dtype != torch.float32:
        raise InvalidArgument(f"{name} must be float32, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise InvalidArgument(f"{name} has shape {list(t.shape)}, expected {list(shape)}")
    return t


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------- ops
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[t, :] = float32(table[ids[t], :]) * scale; ids must already be checked against the table."""
    _gpu(table, "embedding table")
    T = ids.numel()
    V, D = table.shape
    _i32(ids, "token ids")
    _f32(out, "embedding output", (T, D))
    _call(_lib("elementwise").tie_embed, "embed", table.data_ptr(), _code(table, "embedding table"), ids.data_ptr(),
                                         out.data_ptr(), T, D, float(scale), _stream())


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = RMSNorm(x[rows[r]] if rows is given else x[r]) * weight, statistics in float32."""
    _gpu(x, "rms_norm input")
    _gpu(out, "rms_norm output")
    n = x.shape[-1]
    _f32(weight, "rms_norm weight", (n,))
    R = out.numel() // n if n else 0
    if out.shape[-1] != n:
        raise InvalidArgument(f"rms_norm output has width {out.shape[-1]}, input {n}")
    if rows is None:
        if x.numel() != out.numel():
            raise InvalidArgument(f"rms_norm output {list(out.shape)} does not match input {list(x.shape)}")
    else:
        _i32(rows, "rms_norm rows", R)
    _call(_lib("elementwise").tie_rms_norm, "rms_norm", x.data_ptr(), _code(x, "rms_norm input"), weight.data_ptr(), float(eps),
                                            out.data_ptr(), _code(out, "rms_norm output"), _ptr(rows), R, n,
                                            _stream())


def add_partials(x: torch.Tensor, partials: torch.Tensor, weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                 out: Optional[torch.Tensor] = None) -> None:
    """x += partials[0] + partials[1] + ... (float32, in plane order); with ``weight``, out = RMSNorm(x) * weight too.

    ``partials`` is the ``[S, R, n]`` output of a product cut along K (``skinny_gemm_bf16(splits=S)``).
    """
    _gpu(x, "partial sums' target")
    _gpu(partials, "partial sums")
    if x.dtype != torch.float32 or partials.dtype != torch.float32 or partials.dim() != 3 or x.dim() != 2 or \
            tuple(partials.shape[1:]) != tuple(x.shape):
        raise InvalidArgument(f"add_partials: target {list(x.shape)} {x.dtype}, partial sums {list(partials.shape)} "
                              f"{partials.dtype}; both must be float32 and the planes shaped like the target")
    R, n = x.shape
    code = F32
    if weight is not None:
        _f32(weight, "rms_norm weight", (n,))
        _gpu(out, "rms_norm output")
        if tuple(out.shape) != (R, n):
            raise InvalidArgument(f"rms_norm output {list(out.shape)} does not match input {[R, n]}")
        code = _code(out, "rms_norm output")
    _call(_lib("elementwise").tie_add_partials_rms_norm, "add_partials",
        x.data_ptr(), partials.data_ptr(), R * n, partials.shape[0], _ptr(weight), float(eps), _ptr(out), code, R, n,
        _stream())


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu") -> None:
    """out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i] for gate_up of shape [T, 2I]; ``activation`` "silu" or
    "gelu_tanh" (``0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))``)."""
    if activation not in GATE_ACTIVATIONS:
        raise InvalidArgument(f"a gate's activation is one of {', '.join(GATE_ACTIVATIONS)}, not '{activation}'")
    _gpu(gate_up, "swiglu input")
    _gpu(out, "swiglu output")
    T, two_i = gate_up.shape
    if two_i % 2 or tuple(out.shape) != (T, two_i // 2):
        raise InvalidArgument(f"swiglu: input {list(gate_up.shape)} and output {list(out.shape)} do not match")
    _call(_lib("elementwise").tie_swiglu, "swiglu", gate_up.data_ptr(), _code(gate_up, "swiglu input"), out.data_ptr(),
                                          _code(out, "swiglu output"), T, two_i // 2, GATE_ACTIVATIONS[activation],
                                          _stream())


def gelu(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = 0.5 x (1 + erf(x / sqrt 2)), the exact gelu, element by element in float32."""
    _gpu(x, "gelu input")
    _gpu(out, "gelu output")
    if x.numel() != out.numel():
        raise InvalidArgument("gelu: sizes differ")
    _call(_lib("elementwise").tie_gelu, "gelu", x.data_ptr(), _code(x, "gelu input"), out.data_ptr(),
          _code(out, "gelu output"), x.numel(), _stream())


def poly_norm(z: torch.Tensor, coeff: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = a N(z) + b N(z^2) + c N(z^3) + e row by row, powers element by element, N(y) = y / sqrt(mean(y^2) + eps);
    ``coeff`` holds (a, b, c, e) as float32 on the device. ``z`` float32 rows, ``out`` float32 or bfloat16."""
    _f32(z, "poly_norm input")
    _gpu(out, "poly_norm output")
    _f32(coeff, "poly_norm coefficients", (4,))
    if z.dim() != 2 or tuple(out.shape) != tuple(z.shape):
        raise InvalidArgument(f"poly_norm output {list(out.shape)} does not match input {list(z.shape)}")
    _call(_lib("elementwise").tie_poly_norm, "poly_norm", z.data_ptr(), F32, coeff.data_ptr(), float(eps),
          out.data_ptr(), _code(out, "poly_norm output"), z.shape[0], z.shape[1], _stream())


def scale_softcap(x: torch.Tensor, scale: float = 1.0, cap: Optional[float] = None) -> None:
    """x <- cap * tanh(x * scale / cap) in place, float32; without a cap only the scale."""
    _f32(x, "logits")
    _call(_lib("elementwise").tie_scale_softcap, "scale_softcap", x.data_ptr(), x.numel(), float(scale),
          float(cap or 0.0), _stream())


class RoutedParts:
    """A routed feed-forward's result before it is combined: the chosen experts' results by place
    (``parts`` float32 ``[slots, n]``), each row's places (``where`` int32 ``[T, top]``, -1 for an expert that returns
    its input), weights (float32 ``[T, top]``) and the input rows themselves (``self_rows`` ``[T, n]``)."""

    __slots__ = ("parts", "where", "weights", "self_rows")

    def __init__(self, parts, where, weights, self_rows):
        self.parts, self.where, self.weights, self.self_rows = parts, where, weights, self_rows


def norm_add_norm(y, w_post: torch.Tensor, eps_post: float, x: torch.Tensor, w_next: Optional[torch.Tensor] = None,
                  eps_next: float = 0.0, out: Optional[torch.Tensor] = None) -> None:
    """``x += RMSNorm(y) * w_post`` and, with ``w_next``, ``out = RMSNorm(x) * w_next`` of the updated rows, one pass.

    ``y`` is a sub-layer's result: float32 ``[T, n]``, planes of partial sums ``[S, T, n]`` (added in plane
    order), or a ``RoutedParts`` still to be combined. ``x`` is the float32 stream ``[T, n]``.
    """
    _f32(x, "the stream")
    T, n = x.shape
    _f32(w_post, "norm weight", (n,))
    y_ptr, stride, count = None, 0, 1
    parts = where = weights = self_rows = None
    self_code, top = F32, 1
    if isinstance(y, RoutedParts):
        parts, where, weights, self_rows = y.parts, y.where, y.weights, y.self_rows
        _f32(parts, "the experts' results")
        _i32(where, "places")
        _f32(weights, "routing weights")
        _gpu(self_rows, "the feed-forward's input rows")
        top = where.shape[1]
        if parts.shape[-1] != n or tuple(where.shape) != (T, top) or tuple(weights.shape) != (T, top) or \
                tuple(self_rows.shape) != (T, n):
            raise InvalidArgument("norm_add_norm: the routed parts do not fit the stream")
        self_code = _code(self_rows, "the feed-forward's input rows")
    else:
        _f32(y, "the sub-layer's result")
        if y.dim() == 3:
            count = y.shape[0]
            stride = T * n
        if tuple(y.shape[-2:]) != (T, n):
            raise InvalidArgument(f"norm_add_norm: result {list(y.shape)} does not fit the stream {[T, n]}")
        y_ptr = y.data_ptr()
    code = F32
    if w_next is not None:
        _f32(w_next, "next norm weight", (n,))
        _gpu(out, "next norm output")
        if tuple(out.shape) != (T, n):
            raise InvalidArgument(f"next norm output {list(out.shape)} does not match {[T, n]}")
        code = _code(out, "next norm output")
    if n > 15360:
        raise InvalidArgument(f"norm_add_norm keeps a row of at most 15360 values in LDS, got {n}")
    _call(_lib("elementwise").tie_norm_add_norm, "norm_add_norm", y_ptr, stride, count, _ptr(parts), _ptr(where),
          _ptr(weights), _ptr(self_rows), self_code, top, w_post.data_ptr(), float(eps_post), x.data_ptr(),
          _ptr(w_next), float(eps_next), _ptr(out), code, T, n, _stream())


def cast(x: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(x, "cast input")
    _gpu(out, "cast output")
    if x.numel() != out.numel():
        raise InvalidArgument("cast: sizes differ")
    _call(_lib("elementwise").tie_cast, "cast", x.data_ptr(), _code(x, "cast input"), out.data_ptr(),
                                        _code(out, "cast output"), x.numel(), _stream())


def take_tokens(tokens: torch.Tensor, sources: torch.Tensor, previous: torch.Tensor) -> None:
    """``tokens[i] = previous[sources[i]]`` where ``sources[i] >= 0`` (all int32 on the device): the rows of a step
    whose token an earlier step's sampling left on the GPU, unread by the host."""
    T = tokens.numel()
    _i32(tokens, "tokens")
    _i32(sources, "token sources", T)
    _i32(previous, "the earlier step's tokens")
    _call(_lib("elementwise").tie_take_tokens, "take_tokens", tokens.data_ptr(), sources.data_ptr(), previous.data_ptr(),
          T, previous.numel(), _stream())


def add_bias(rows: torch.Tensor, bias: torch.Tensor) -> None:
    """rows[m] += bias, in place (float32 arithmetic; rows float32 or bfloat16, bias float32 ``[width]``)."""
    _gpu(rows, "rows")
    if rows.dim() != 2 or not rows.is_contiguous():
        raise InvalidArgument(f"add_bias takes contiguous rows [M, width], got {list(rows.shape)}")
    _f32(bias, "bias", (rows.shape[1],))
    _call(_lib("elementwise").tie_add_bias, "add_bias", rows.data_ptr(), _code(rows, "rows"), rows.shape[0],
          rows.shape[1], bias.data_ptr(), _stream())


def scale_rows(rows: torch.Tensor, row_scale: "RowScale") -> None:
    """``rows[m] *= 1 / sqrt(row_scale.squares[m].sum() / n + eps)`` in place (bfloat16 or float32): for rows that
    were left without their norm's factor and go to a product that cannot apply it."""
    _gpu(rows, "rows")
    M, n = rows.shape
    _f32(row_scale.squares, "sums of squares")
    if row_scale.squares.dim() != 2 or row_scale.squares.shape[0] < M or not row_scale.squares.is_contiguous():
        raise InvalidArgument(f"sums of squares {list(row_scale.squares.shape)} do not cover {M} rows")
    _call(_lib("elementwise").tie_scale_rows, "scale_rows", rows.data_ptr(), _code(rows, "rows"), M, n,
          row_scale.squares.data_ptr(), row_scale.squares.shape[1], float(row_scale.n), float(row_scale.eps), _stream())


def random_fill(out: torch.Tensor, key: int, kind: str, scale: float) -> None:
    """Fills float32 ``out`` with the random weights of the stream ``key``: element i depends on (key, i) alone
    and equals, bit for bit, what ``weights.random_init`` draws on the host. ``kind``: "normal" (``scale`` the
    standard deviation) or "one_plus_uniform" (1 + U(-scale, scale))."""
    _f32(out, "random output")
    if not out.is_contiguous():
        raise InvalidArgument("random_fill needs a contiguous tensor")
    kinds = {"normal": 0, "one_plus_uniform": 1}
    if kind not in kinds:
        raise InvalidArgument(f"random_fill draws 'normal' or 'one_plus_uniform', not '{kind}'")
    if out.numel():
        _call(_lib("elementwise").tie_random_fill, "random_fill", out.data_ptr(), out.numel(), int(key) & (2 ** 64 - 1),
              kinds[kind], float(scale), _stream())


def stream_read(data: torch.Tensor, sink: torch.Tensor, workgroups: int = 2048) -> int:
    """Launches a kernel that reads ``data`` once, in consecutive runs a wave; returns the bytes it reads (whole
    chunks of 8 KB a wave). For measuring what a streaming read of cold memory reaches: the caller times it."""
    _gpu(data, "data")
    _i32(sink, "sink")
    read = ctypes.c_longlong(0)
    _call(_lib("machine_peaks").tie_stream_read, "stream_read", data.data_ptr(), data.numel() * data.element_size(),
          int(workgroups), sink.data_ptr(), ctypes.addressof(read), _stream())
    return int(read.value)


def mfma_rate(sink: torch.Tensor, workgroups: int = 1024, rounds: int = 4096) -> float:
    """Launches a kernel of bfloat16 matrix instructions on registers alone; returns its floating-point operations.
    For measuring the rate the matrix cores sustain: the caller times it."""
    _f32(sink, "sink")
    flops = ctypes.c_double(0.0)
    _call(_lib("machine_peaks").tie_mfma_rate, "mfma_rate", int(workgroups), int(rounds), sink.data_ptr(),
          ctypes.addressof(flops), _stream())
    return float(flops.value)


def gemm_generic(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out (+)= x @ w.T with float32 multiply-adds; operands float32 or bfloat16 in any mix."""
    _gpu(x, "matmul input")
    _gpu(w, "matmul weight")
    _gpu(out, "matmul output")
    T, K = x.shape
    N, K2 = w.shape
    if K != K2 or tuple(out.shape) != (T, N):
        raise InvalidArgument(f"matmul: input {list(x.shape)}, weight {list(w.shape)}, output {list(out.shape)}")
    _call(_lib("gemm_generic").tie_gemm_generic, "gemm_generic",
        x.data_ptr(), _code(x, "matmul input"), w.data_ptr(), _code(w, "matmul weight"), out.data_ptr(),
        _code(out, "matmul output"), int(accumulate), T, N, K, _stream())


class PackedWeight:
    """A bfloat16 ``[N, K]`` weight stored as ``[N/16][K/32]`` blocks of 1 KB in the matrix cores' operand order.

    Block (t, b) holds rows 16 t .. 16 t + 15 over k = 32 b .. 32 b + 31; within it the 8 elements of
    (row r, k-chunk c) lie at element (16 c + r) * 8. A wave of the decode product then loads 1 KB of
    consecutive memory per matrix instruction and walks K as one contiguous run, and the tiled product
    stages one block per load. Built once at load time by ``pack_weight``; only the bfloat16 products
    read it (``N % 16 == 0`` and ``K % 32 == 0``).
    """

    __slots__ = ("blocks", "shape")
    dtype = torch.bfloat16

    def __init__(self, blocks: torch.Tensor, shape):
        self.blocks = blocks
        self.shape = tuple(shape)

    def data_ptr(self) -> int:
        return self.blocks.data_ptr()

    @property
    def device(self):
        return self.blocks.device

    def unpacked(self) -> torch.Tensor:
        """The ``[N, K]`` row-major matrix again (a copy)."""
        N, K = self.shape
        return self.blocks.view(N // 16, K // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(N, K).contiguous()


def packable(w) -> bool:
    """Whether ``pack_weight`` takes this matrix: bfloat16, on the GPU, rows in steps of 16 and K in steps of 32.

    K between 96 and 2^22 is what the tiled product's packed path takes (at least three slices of 32; the
    row offsets of a tile within 32 bits).
    """
    return isinstance(w, torch.Tensor) and w.is_cuda and w.dim() == 2 and w.dtype == torch.bfloat16 and \
        w.shape[0] % 16 == 0 and w.shape[1] % 32 == 0 and 96 <= w.shape[1] <= (1 << 22)


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """The matrix in the blocked layout of ``PackedWeight`` (a copy; the row-major tensor can be dropped)."""
    if not packable(w):
        raise InvalidArgument(f"pack_weight takes a bfloat16 GPU matrix [N % 16 == 0, K % 32 == 0, K >= 96], got "
                              f"{list(w.shape)} {w.dtype}")
    N, K = w.shape
    blocks = w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(N, K)
    return PackedWeight(blocks, (N, K))


def _bf16_product_operands(x, w, out, gated, what):
    _gpu(x, "matmul input")
    _gpu(w.blocks if isinstance(w, PackedWeight) else w, "matmul weight")
    _gpu(out, "matmul output")
    M, K = x.shape
    N, K2 = w.shape
    width = N // 2 if gated else N
    if K != K2 or tuple(out.shape) != (M, width):
        raise InvalidArgument(f"matmul: input {list(x.shape)}, weight {list(w.shape)}, output {list(out.shape)}")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise InvalidArgument(f"{what} takes bfloat16 operands")
    if K % 8:
        raise InvalidArgument(f"{what} takes K % 8 == 0, got K={K}")
    if gated and (N % 16 or out.dtype != torch.bfloat16):
        raise InvalidArgument(f"{what}: a gated product needs N % 16 == 0 and a bfloat16 output")
    return M, N, K


def skinny_splits(N: int, K: int) -> int:
    """Ranges of K a decode-time product of up to 16 rows over a ``[N, K]`` weight is best cut into when its caller
    adds partial sums."""
    return int(_lib("skinny_gemm_bf16").tie_skinny_gemm_splits(N, K))


@functools.lru_cache(maxsize=None)
def few_rows_plan(M: int, N: int, K: int, gated: bool = False) -> tuple:
    """``(shares_x, tiles, splits)`` of the decode product for ``M`` rows over a packed ``[N, K]`` weight: whether the
    kernel that shares x through LDS runs (17 to 64 rows), the weight tiles a workgroup takes, and the ranges of K
    the product is best cut into when its caller adds partial sums (up to 16 rows: ``skinny_splits``)."""
    shares_x, tiles = ctypes.c_int(0), ctypes.c_int(0)
    splits = int(_lib("skinny_gemm_bf16").tie_skinny_few_rows_plan(M, N, K, int(gated), ctypes.addressof(shares_x),
                                                                  ctypes.addressof(tiles)))
    return bool(shares_x.value), tiles.value, splits


NORM_EPILOGUE_ROWS = 16      # rows up to which the decode product's epilogue does the norms' work (SkNorm)
# Whether steps of up to that many rows leave the RMS norms between their sub-layers to the products' epilogues
# (parts.Linear.prepares_norms). False: every norm is a kernel of its own (tests compare the two ways).
NORMS_IN_PRODUCTS = True


class RowScale:
    """Rows that are a norm's input times its weight, the ``1 / rms`` still to come: ``squares[m]`` holds, per
    16-column tile of the row the norm saw, the sum of its squares; the factor is
    ``1 / sqrt(squares[m].sum() / n + eps)`` and belongs on whatever product is formed from the rows."""

    __slots__ = ("squares", "n", "eps")

    def __init__(self, squares: torch.Tensor, n: int, eps: float):
        self.squares, self.n, self.eps = squares, int(n), float(eps)


def skinny_gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
                     gated: bool = False, splits: int = 1, row_scale: Optional[RowScale] = None,
                     next_norm: Optional[tuple] = None, tiles: int = 0, loads: int = 0, waves: int = 0) -> None:
    """out (+)= x @ w.T for at most 64 rows of bfloat16 x against bfloat16 w, on the matrix cores.

    ``gated``: w is a gate/up pair interleaved by ``interleave_gate_up`` and out receives silu(gate) * up.
    ``splits`` > 1: out is ``[splits, M, N]`` float32 and receives one plane of partial sums per range
    of K, for the consumer to add (``add_partials``, or a kernel that takes planes).
    Up to ``NORM_EPILOGUE_ROWS`` rows the epilogue can do the work of the RMS norms around the product:
    ``row_scale``: x lacks its norm's ``1 / rms``, and the sums are multiplied by it (before the activation of
    a gated product); ``next_norm = (weight [N], next_x bfloat16 [M, N], squares float32 [M, N / 16])`` with
    ``accumulate`` and one plane: out is the residual stream, and beside ``out += x @ w.T`` the epilogue leaves
    ``next_x = bfloat16(out * weight)`` and the sums of ``out ** 2`` per 16-column tile for the norm that follows
    (a ``RowScale`` for whoever multiplies ``next_x``).
    """
    if splits > 1:
        if out.dim() != 3 or out.shape[0] != splits or out.dtype != torch.float32 or accumulate or gated:
            raise InvalidArgument(f"skinny_gemm_bf16: {splits} splits need a float32 output of {splits} planes, "
                                  f"got {list(out.shape)} {out.dtype}, and neither accumulate nor gated")
        M, N, K = _bf16_product_operands(x, w, out[0], gated, "skinny_gemm_bf16")
    else:
        M, N, K = _bf16_product_operands(x, w, out, gated, "skinny_gemm_bf16")
    if M > 64:
        raise InvalidArgument(f"skinny_gemm_bf16 takes at most 64 rows, got {M}")
    if gated and accumulate:
        raise InvalidArgument("a gated product does not accumulate")
    if row_scale is None and next_norm is None:
        _call(_lib("skinny_gemm_bf16").tie_skinny_gemm_bf16, "skinny_gemm_bf16",
            x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"), int(accumulate), int(gated), M, N, K,
            int(splits), int(isinstance(w, PackedWeight)), _stream())
        return
    if M > NORM_EPILOGUE_ROWS:
        raise InvalidArgument(f"the product's epilogue does the norms' work for up to {NORM_EPILOGUE_ROWS} rows, not {M}")
    squares_in, tiles_in, n_in, eps_in = None, 0, 1.0, 0.0
    if row_scale is not None:
        _f32(row_scale.squares, "sums of squares")
        if row_scale.squares.dim() != 2 or row_scale.squares.shape[0] < M or not row_scale.squares.is_contiguous() \
                or row_scale.n <= 0:
            raise InvalidArgument(f"sums of squares {list(row_scale.squares.shape)} do not cover {M} rows")
        squares_in, tiles_in, n_in, eps_in = row_scale.squares, row_scale.squares.shape[1], float(row_scale.n), row_scale.eps
    next_w = next_x = squares_out = None
    if next_norm is not None:
        next_w, next_x, squares_out = next_norm
        _f32(next_w, "the next norm's weight", (N,))
        _f32(squares_out, "sums of squares", (M, N // 16))
        _gpu(next_x, "the next norm's rows")
        if splits != 1 or gated or not accumulate or out.dtype != torch.float32 or N % 16 or \
                next_x.dtype != torch.bfloat16 or tuple(next_x.shape) != (M, N) or not next_x.is_contiguous() or \
                not squares_out.is_contiguous():
            raise InvalidArgument("a product that prepares the next norm adds to a float32 stream in one plane, is not "
                                  f"gated, and leaves bfloat16 rows [{M}, {N}] (N in steps of 16)")
    _call(_lib("skinny_gemm_bf16").tie_skinny_gemm_bf16_norm, "skinny_gemm_bf16_norm",
        x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"), int(accumulate), int(gated), M, N, K,
        int(splits), int(isinstance(w, PackedWeight)), _ptr(squares_in), tiles_in, n_in, eps_in, _ptr(next_w),
        _ptr(next_x), _ptr(squares_out), int(tiles), int(loads), int(waves), _stream())


def gemm_splits(M: int, N: int, K: int, packed: bool = False) -> int:
    """Ranges of K a product of M > 64 rows over a ``[N, K]`` weight is best cut into when its caller adds partial sums."""
    return int(_lib("gemm_bf16").tie_gemm_bf16_splits(M, N, K, int(packed)))


def gemm_tile(M: int, N: int, K: int, packed: bool = False, splits: int = 0) -> int:
    """The tile (``gemm_bf16``'s numbering) a product left to choose runs on, with ``splits`` ranges of K fixed (0: the plan's own)."""
    return int(_lib("gemm_bf16").tie_gemm_bf16_tile(M, N, K, int(packed), splits))


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, tile: int = 0,
              gated: bool = False, splits: int = 1) -> None:
    """out (+)= x @ w.T for bfloat16 operands on the matrix cores, any number of rows; K % 8 == 0.

    ``tile`` picks the workgroup tile (1 = 128x128, 2 = 256x256, 3 = 256x128; 4 = 256x256, 5 = 256x128, 6 = 128x256,
    7 = 128x128, 8 = 64x256, 9 = 64x128 and 10 = 256x192 with operand slices loaded straight into LDS, which need
    K % 32 == 0 and N % 4 == 0; 0 lets the kernel choose);
    ``gated`` and ``splits`` as in ``skinny_gemm_bf16`` (planes of partial sums, ``[splits, M, N]`` float32).
    """
    if splits > 1:
        if out.dim() != 3 or out.shape[0] != splits or out.dtype != torch.float32 or accumulate or gated:
            raise InvalidArgument(f"gemm_bf16: {splits} splits need a float32 output of {splits} planes, got "
                                  f"{list(out.shape)} {out.dtype}, and neither accumulate nor gated")
        M, N, K = _bf16_product_operands(x, w, out[0], gated, "gemm_bf16")
    else:
        M, N, K = _bf16_product_operands(x, w, out, gated, "gemm_bf16")
    if accumulate and (gated or out.dtype != torch.float32):
        raise InvalidArgument("gemm_bf16 accumulates into float32 outputs only, and not in a gated product")
    _call(_lib("gemm_bf16").tie_gemm_bf16, "gemm_bf16", x.data_ptr(), w.data_ptr(), out.data_ptr(), _code(out, "matmul output"),
                                           int(accumulate), int(gated), M, N, K, tile, int(splits),
                                           int(isinstance(w, PackedWeight)), _stream())


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The weight layout of a gated product: blocks of 16 rows = 8 gate rows then the 8 up rows of the same outputs."""
    I, K = gate.shape
    if up.shape != gate.shape or I % 8:
        raise InvalidArgument(f"gate {list(gate.shape)} and up {list(up.shape)} must match, with a multiple of 8 rows")
    return torch.stack([gate.reshape(I // 8, 8, K), up.reshape(I // 8, 8, K)], dim=1).reshape(2 * I, K).contiguous()


_few_rows_memo: Dict[tuple, bool] = {}


def decode_product_rows(M: int, w, gated: bool = False) -> bool:
    """Whether ``M`` rows against ``w`` go to the decode product (``skinny_gemm_bf16``) rather than the tiled one.

    Up to 32 rows always, above 64 never; between, the tiled product with 64-row tiles where it takes the weight
    (packed, whole slices of K), except for gated products that are not very wide (measured).
    """
    if M <= 32 or M > 64:
        return M <= 32
    N, K = w.shape
    packed = isinstance(w, PackedWeight)
    key = (M, N, K, packed, bool(gated))
    tiled = _few_rows_memo.get(key)
    if tiled is None:
        tiled = _few_rows_memo[key] = bool(_lib("gemm_bf16").tie_gemm_bf16_wins_few_rows(M, N, K, int(packed), int(gated)))
    return not tiled


def linear_swiglu(x: torch.Tensor, w_interleaved: torch.Tensor, out: torch.Tensor,
                  row_scale: Optional[RowScale] = None, activation: str = "silu") -> None:
    """out = act(x @ gate.T) * (x @ up.T) in one product over the interleaved weight; bfloat16 only.
    ``row_scale`` as in ``skinny_gemm_bf16`` (up to ``NORM_EPILOGUE_ROWS`` rows); ``activation`` "silu" or
    "gelu_tanh"."""
    gated = 1 + GATE_ACTIVATIONS[activation]
    if decode_product_rows(x.shape[0], w_interleaved, gated=True):
        skinny_gemm_bf16(x, w_interleaved, out, gated=gated, row_scale=row_scale)
    elif row_scale is not None:
        raise InvalidArgument(f"{x.shape[0]} rows without their norm's factor: only the decode product applies it")
    else:
        gemm_bf16(x, w_interleaved, out, gated=gated)


@functools.lru_cache(maxsize=None)
def norm_epilogue_rows(N: int, K: int) -> int:
    """The most rows for which a product over a packed ``[N, K]`` weight that ends a sub-layer is worth running
    with the next norm's work in its epilogue (``skinny_gemm_bf16(next_norm=...)``) rather than as planes that a
    norm kernel adds; 0 where it never is. Never above ``NORM_EPILOGUE_ROWS``."""
    return min(NORM_EPILOGUE_ROWS, int(_lib("skinny_gemm_bf16").tie_skinny_norm_epilogue_rows(N, K)))


def applies_row_scale(x: torch.Tensor, w) -> bool:
    """Whether ``linear`` / ``linear_swiglu`` over these operands run on the product whose epilogue applies a
    ``RowScale`` (the decode product, up to ``NORM_EPILOGUE_ROWS`` rows)."""
    # the kernel holds the tiles' sums of squares of all rows in 32 KB of LDS, 64 tiles (256 bytes) a load
    staged = x.shape[0] * (-(-(x.shape[1] // 16) // 64)) * 256
    return x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 16 == 0 and \
        x.shape[0] <= NORM_EPILOGUE_ROWS and staged <= 32768


def linear(x: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False, row_scale: Optional[RowScale] = None) -> None:
    """out (+)= x @ w.T, on the fastest kernel that takes these operands (w a matrix or a ``PackedWeight``).
    ``row_scale``: see ``skinny_gemm_bf16``; only where ``applies_row_scale`` says so."""
    if row_scale is not None and not (applies_row_scale(x, w) and not (accumulate and out.dtype != torch.float32)):
        raise InvalidArgument("these operands do not run on the product that applies a row scale: scale the rows first")
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and \
            not (accumulate and out.dtype != torch.float32):
        if decode_product_rows(x.shape[0], w):
            skinny_gemm_bf16(x, w, out, accumulate, row_scale=row_scale)
        else:
            gemm_bf16(x, w, out, accumulate)
    elif isinstance(w, PackedWeight):
        raise InvalidArgument(f"a packed weight is read by the bfloat16 products only: input {x.dtype}, output "
                              f"{out.dtype}, accumulate={accumulate}")
    else:
        gemm_generic(x, w, out, accumulate)


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor, amplitude: float = 1.0) -> None:
    """out[t] = amplitude * [cos(float(positions[t]) * inv_freq), sin(...)]: the rotation table of one step,
    ``[T, 2 * half]`` float32."""
    T = positions.numel()
    half = inv_freq.numel()
    _i32(positions, "positions", T)
    _f32(inv_freq, "inv_freq", (half,))
    _f32(out, "rope angles", (T, 2 * half))
    _call(_lib("elementwise").tie_rope_angles, "rope_angles", positions.data_ptr(), inv_freq.data_ptr(), out.data_ptr(), T, half,
                                               float(amplitude), _stream())


def qk_norm_rope_kv_write(qkv: torch.Tensor, q_out: torch.Tensor, q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], eps: float, inv_freq: Optional[torch.Tensor],
                          positions: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                          v_cache: Optional[torch.Tensor], num_heads: int, num_kv_heads: int, head_dim: int,
                          block_size: int, write_kv: bool = True, k_dense: Optional[torch.Tensor] = None,
                          planes: int = 1, plane_stride: int = 0, angles: Optional[torch.Tensor] = None,
                          rotary_dim: Optional[int] = None, pairing: str = "rotate_half",
                          value_mix: Optional[tuple] = None, values_are_keys: bool = False,
                          bias: Optional[torch.Tensor] = None) -> None:
    """Per-head RMSNorm of q and k, rotation by position, q to ``q_out``, k and v into the paged cache.

    The first ``rotary_dim`` dimensions of a head (default: all) are rotated, as pairs
    ``(i, i + rotary_dim / 2)`` (``pairing`` "rotate_half") or ``(2 i, 2 i + 1)`` ("interleaved") by
    ``position * inv_freq[i]``; ``inv_freq`` holds ``rotary_dim / 2`` values.

    ``angles`` (from ``rope_angles`` for the same positions and ``inv_freq``) spares the kernel the
    sines and cosines.

    With ``planes`` > 1, ``qkv`` is the first of that many planes of partial sums, ``plane_stride``
    elements apart, which are added as they are read.

    ``qkv`` is ``[T, >= (H + 2 KVH) * Dh]`` (rows may be wider than what is read). ``q_out`` is a
    ``[T, H * Dh]`` tensor or a view into ``qkv`` itself (rows ``qkv.stride(0)`` apart). With
    ``k_dense`` (``[T, KVH * Dh]`` or a view into ``qkv``) the keys go there instead of the cache
    and ``write_kv`` must be off. Null weights or ``inv_freq`` skip the norm or the rotation.

    ``value_mix`` blends values across layers before they are cached: ``("keep", first)`` stores this layer's values
    of the step's tokens in ``first`` (float32 ``[T, KVH * width]``, ``width <= Dh``: the leading dimensions of every
    value head, the others being padding), ``("blend", first, lam)`` caches ``(1 - lam) * v + lam * first`` with
    ``lam`` one float32 on the device.

    ``values_are_keys``: the rows hold no value heads, ``[q | k]`` only; what is cached as values are the keys as
    projected, before norm and rotation.

    ``bias`` (float32, one value per column the kernel reads of a row: ``[q | k | v]`` or ``[q | k]``): the
    projection's bias, added as the sums are read, so that the product needs no pass of its own for it.
    """
    _gpu_strided(qkv, "qkv")
    _gpu_strided(q_out, "q output")
    T, in_width = qkv.shape
    in_row = qkv.stride(0)
    H, KVH, Dh = num_heads, num_kv_heads, head_dim
    heads = H + (KVH if (write_kv or k_dense is not None) else 0) + (KVH if write_kv and not values_are_keys else 0)
    if in_width < heads * Dh:
        raise InvalidArgument(f"qkv rows hold {in_width} values, {heads * Dh} are needed")
    if tuple(q_out.shape) != (T, H * Dh):
        raise InvalidArgument(f"q output has shape {list(q_out.shape)}, expected {[T, H * Dh]}")
    if Dh % 2 or Dh > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {Dh} must be even and at most {MAX_HEAD_DIM}")
    if T > MAX_STEP_TOKENS:
        raise InvalidArgument(f"a step of {T} tokens exceeds the {MAX_STEP_TOKENS} this kernel takes")
    for wt, nm in ((q_weight, "q_norm weight"), (k_weight, "k_norm weight")):
        if wt is not None:
            _f32(wt, nm, (Dh,))
    rotary_dim = Dh if rotary_dim is None else int(rotary_dim)
    if rotary_dim % 2 or not 0 <= rotary_dim <= Dh:
        raise InvalidArgument(f"rotary_dim {rotary_dim} must be even and at most head_dim {Dh}")
    if pairing not in ("rotate_half", "interleaved"):
        raise InvalidArgument(f"the fused kernel rotates pairs as 'rotate_half' or 'interleaved', not '{pairing}'")
    if inv_freq is not None:
        _f32(inv_freq, "inv_freq", (rotary_dim // 2,))
    if angles is not None:
        _f32(angles, "rope angles", (T, rotary_dim))
    _i32(positions, "positions", T)
    cache_code = _code(q_out, "q output")
    k_row = 0
    if k_dense is not None:
        if write_kv:
            raise InvalidArgument("keys go either to k_dense or into the cache, not both")
        _gpu_strided(k_dense, "k output")
        if tuple(k_dense.shape) != (T, KVH * Dh) or k_dense.dtype != q_out.dtype:
            raise InvalidArgument(f"k output {list(k_dense.shape)} {k_dense.dtype} does not fit {[T, KVH * Dh]}")
        k_row = k_dense.stride(0)
    if write_kv:
        _i32(slots, "slot mapping", T)
        _gpu(k_cache, "k cache")
        _gpu(v_cache, "v cache")
        _check_cache(k_cache, v_cache, KVH, block_size, Dh)
        cache_code = _cache_code(k_cache, q_out, "k cache")
    v_first = v_lambda = None
    v_mode = v_width = 0
    if value_mix is not None:
        if not write_kv or value_mix[0] not in ("keep", "blend"):
            raise InvalidArgument("values are blended on their way into the cache: ('keep', first) or ('blend', first, lam)")
        v_first = _f32(value_mix[1], "the first layer's values")
        v_width = v_first.shape[-1] // KVH
        if v_first.dim() != 2 or v_first.shape[0] != T or v_first.shape[1] != KVH * v_width or not 0 < v_width <= Dh:
            raise InvalidArgument(f"the first layer's values {list(v_first.shape)} do not fit {T} rows of {KVH} heads of "
                                  f"at most {Dh}")
        v_mode = 1
        if value_mix[0] == "blend":
            v_lambda = _f32(value_mix[2], "the blend weight")
            if v_lambda.numel() != 1:
                raise InvalidArgument("the blend weight is one number")
            v_mode = 2
    _call(_lib("elementwise").tie_qk_norm_rope_kv_write, "qk_norm_rope_kv_write",
        qkv.data_ptr(), _code(qkv, "qkv"), q_out.data_ptr(), _code(q_out, "q output"), _ptr(q_weight),
        _ptr(k_weight), float(eps), _ptr(inv_freq), _ptr(angles), positions.data_ptr(),
        _ptr(slots) if write_kv else None,
        _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None, cache_code, int(write_kv),
        _ptr(k_dense), T, H, KVH, Dh, block_size, in_row, q_out.stride(0), k_row, int(plane_stride), int(planes),
        rotary_dim, int(pairing == "interleaved"), _ptr(v_first), _ptr(v_lambda), v_mode, v_width,
        int(bool(values_are_keys)), _ptr(_f32(bias, "projection bias", (heads * Dh,)) if bias is not None else None),
        _stream())


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                            query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                            seq_of_row: torch.Tensor, num_heads: int, scale: float,
                            window: Optional[int] = None, softcap: Optional[float] = None,
                            chunk: Optional[int] = None, sinks: Optional[torch.Tensor] = None,
                            keep_first: int = 0) -> None:
    """Causal attention of every query row over its sequence's cached keys (float32 arithmetic, any sizes).

    ``softcap`` c (None or 0: none): scores become ``c * tanh(scale * q.k / c)`` before the softmax.
    ``chunk`` n: a query at position p reads the keys from ``p - p % n`` on (causal chunks counted from the
    sequence's position 0) instead of a sliding ``window``. ``sinks`` (float32 ``[heads]``): ``exp(sinks[h])``
    is one more term of head h's softmax denominator. ``keep_first`` f (beside a window): the keys of positions
    below f are read as well, at their true positions."""
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    T = q.shape[0]
    H = num_heads
    if tuple(q.shape) != (T, H * Dh) or tuple(out.shape) != (T, H * Dh):
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if H % KVH:
        raise InvalidArgument(f"{H} query heads are not a multiple of {KVH} kv heads")
    if Dh > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {Dh} exceeds the {MAX_HEAD_DIM} this kernel takes")
    if T > MAX_STEP_TOKENS:
        raise InvalidArgument(f"a step of {T} tokens exceeds the {MAX_STEP_TOKENS} this kernel takes")
    S = context_lens.numel()
    _i32(query_start, "query_start", S + 1)
    _i32(context_lens, "context_lens")
    _i32(seq_of_row, "seq_of_row", T)
    _i32(block_tables, "block tables")
    if block_tables.dim() != 2 or block_tables.shape[0] < S:
        raise InvalidArgument(f"block tables {list(block_tables.shape)} do not cover {S} sequences")
    if window and chunk:
        raise InvalidArgument("attention takes a sliding window or causal chunks, not both")
    if keep_first and not window:
        raise InvalidArgument("first positions are kept beside a sliding window only")
    if sinks is not None:
        _f32(sinks, "attention sinks", (H,))
    _call(_lib("attention_generic").tie_paged_attention_generic, "paged_attention_generic",
        q.data_ptr(), _code(q, "queries"), k_cache.data_ptr(), v_cache.data_ptr(), _cache_code(k_cache, q, "k cache"),
        out.data_ptr(), _code(out, "attention output"), query_start.data_ptr(), context_lens.data_ptr(),
        block_tables.data_ptr(), seq_of_row.data_ptr(), T, H, KVH, Dh, bs, block_tables.shape[1], float(scale),
        float(softcap or 0.0), int(window or 0), int(chunk or 0), int(keep_first or 0), _ptr(sinks), _stream())


_argmax_workspace = {}


def argmax_rows(logits: torch.Tensor, out: torch.Tensor, max_out: Optional[torch.Tensor] = None) -> None:
    """out[r] = lowest index of the maximum of logits[r]; -1 marks a row with a NaN. ``max_out[r]`` = that maximum."""
    _f32(logits, "logits")
    R, V = logits.shape
    _i32(out, "argmax output", R)
    if max_out is not None:
        _f32(max_out, "row maxima", (R,))
    key = str(logits.device)
    ws = _argmax_workspace.get(key)
    if ws is None or ws[0].numel() < R * 64:
        rows = max(R, 64)
        ws = _argmax_workspace[key] = (torch.empty(rows * 64, dtype=torch.float32, device=logits.device),
                                       torch.empty(rows * 64, dtype=torch.int32, device=logits.device))
    _call(_lib("elementwise").tie_argmax, "argmax", logits.data_ptr(), out.data_ptr(), _ptr(max_out), ws[0].data_ptr(),
                                          ws[1].data_ptr(), R, V, _stream())


ARGMAX_STATIC_MAX_ROWS = 1024     # TIE_ARGMAX_STATIC_MAX_ROWS of csrc/argmax_static.h


def argmax_rows_static(logits: torch.Tensor, out: torch.Tensor, max_out: Optional[torch.Tensor] = None) -> None:
    """``argmax_rows`` without any allocation: the candidates between its two stages live in a static device array.

    For callers that cannot allocate (stream capture, loops that must stay off the allocator). At most
    ``ARGMAX_STATIC_MAX_ROWS`` rows; calls that may overlap on one GPU race on the shared array.
    """
    _f32(logits, "logits")
    R, V = logits.shape
    _i32(out, "argmax output", R)
    if max_out is not None:
        _f32(max_out, "row maxima", (R,))
    if R > ARGMAX_STATIC_MAX_ROWS:
        raise InvalidArgument(f"argmax_rows_static takes at most {ARGMAX_STATIC_MAX_ROWS} rows (the size of its static "
                              f"scratch array), got {R}")
    with torch.cuda.device(logits.device):
        _call(_lib("elementwise").tie_argmax_static, "argmax_static", logits.data_ptr(), out.data_ptr(), _ptr(max_out), R, V,
                                                     _stream())


MAX_SAMPLED_VOCAB = 1 << 20      # rows the temperature sampling kernel takes (the sums of its pieces fit LDS)


def _row_selection(rows: Optional[torch.Tensor], row_max: Optional[torch.Tensor], R: int) -> int:
    count = 0
    if rows is not None:
        _i32(rows, "row numbers")
        count = rows.numel()
        if not 0 < count <= R:
            raise InvalidArgument(f"{count} row numbers for {R} rows")
    if row_max is not None:
        _f32(row_max, "row maxima", (R,))
    return count


def _uniform_numbers(uniform: torch.Tensor, other_uniform, take_other, drew_none, R: int) -> None:
    for t, name in ((uniform, "uniform numbers"), (other_uniform, "the other uniform numbers")):
        if t is None:
            continue
        _gpu(t, name)
        if t.dtype != torch.float64 or t.numel() != R:
            raise InvalidArgument(f"{name} must be float64, one per row")
    if (take_other is None) != (other_uniform is None):
        raise InvalidArgument("the other uniform numbers and the marks of the rows that take them come together")
    if take_other is not None:
        _i32(take_other, "marks of the rows that take the other number", R)
    if drew_none is not None:
        _i32(drew_none, "marks of the rows that drew nothing", R)


def sample_rows(logits: torch.Tensor, inv_temperature: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor,
                rows: Optional[torch.Tensor] = None, row_max: Optional[torch.Tensor] = None,
                other_uniform: Optional[torch.Tensor] = None, take_other: Optional[torch.Tensor] = None,
                drew_none: Optional[torch.Tensor] = None) -> None:
    """Draws one token per row from softmax(logits * inv_temperature) with the given uniform numbers, walking the
    tokens in index order. ``out[r]`` is -1 for a row with a NaN and -2 for a row that is all -inf. With ``rows``
    (int32 row numbers) only those rows are drawn; the other entries of ``out`` stay as they are. With ``row_max``
    (the rows' maxima) the kernel does not look for them and leaves ``out`` of a row without a finite maximum as
    it is. ``drew_none[r]`` becomes 1 where the row took no uniform number (no finite maximum), else 0;
    where ``take_other[r]`` is not 0 the row's number is ``other_uniform[r]`` (a step queued before the one
    before it is read passes that step's ``drew_none``, and both numbers its stream may be at)."""
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise InvalidArgument("logits must be [rows, vocabulary]")
    R, V = logits.shape
    if V > MAX_SAMPLED_VOCAB:
        raise InvalidArgument(f"the sampling kernel takes rows of up to {MAX_SAMPLED_VOCAB} logits, got {V}")
    _f32(inv_temperature, "inverse temperatures", (R,))
    _uniform_numbers(uniform, other_uniform, take_other, drew_none, R)
    _i32(out, "sample output", R)
    count = _row_selection(rows, row_max, R)
    _call(_lib("elementwise").tie_sample, "sample", logits.data_ptr(), _ptr(row_max), inv_temperature.data_ptr(),
          uniform.data_ptr(), _ptr(other_uniform), _ptr(take_other), _ptr(drew_none), _ptr(rows), count, out.data_ptr(),
          R, V, _stream())


MAX_FILTERED_VOCAB = 1 << 19     # rows the top-k / top-p sampling kernel takes (its integer sums fit 64 bits)


def sample_rows_filtered(logits: torch.Tensor, inv_temperature: torch.Tensor, uniform: torch.Tensor,
                         top_k: torch.Tensor, top_p: torch.Tensor, out: torch.Tensor,
                         rows: Optional[torch.Tensor] = None, row_max: Optional[torch.Tensor] = None,
                         other_uniform: Optional[torch.Tensor] = None, take_other: Optional[torch.Tensor] = None,
                         drew_none: Optional[torch.Tensor] = None) -> None:
    """Draws one token per row with top-k and top-p: ``top_k[r]`` most likely kept (0: all), then the smallest
    prefix by likelihood whose weight reaches ``top_p[r]`` of the total (1: all), one uniform number a row, which
    walks the candidates in the order of likelihood also where neither filter removes any (``sample_rows`` walks
    them in index order, as the rule is without filters).
    ``out[r]`` is -1 for a row with a NaN and -2 for a row that is all -inf. With ``rows`` (int32 row numbers)
    only those rows are drawn; the other entries of ``out`` stay as they are. ``row_max``, ``other_uniform``,
    ``take_other`` and ``drew_none`` as in ``sample_rows``."""
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise InvalidArgument("logits must be [rows, vocabulary]")
    R, V = logits.shape
    if V > MAX_FILTERED_VOCAB:
        raise InvalidArgument(f"the top-k / top-p kernel takes rows of up to {MAX_FILTERED_VOCAB} logits, got {V}")
    _f32(inv_temperature, "inverse temperatures", (R,))
    _f32(top_p, "top_p", (R,))
    _i32(top_k, "top_k", R)
    _uniform_numbers(uniform, other_uniform, take_other, drew_none, R)
    _i32(out, "sample output", R)
    count = _row_selection(rows, row_max, R)
    _call(_lib("sample_filtered").tie_sample_filtered, "sample_filtered", logits.data_ptr(), _ptr(row_max),
          inv_temperature.data_ptr(), uniform.data_ptr(), _ptr(other_uniform), _ptr(take_other), _ptr(drew_none),
          top_k.data_ptr(), top_p.data_ptr(), _ptr(rows), count, out.data_ptr(), R, V, _stream())


# Up to this many workgroups of single decoded rows run in the prefill attention kernel beside a step's prompt
# portions rather than in a launch (and a merge) of the decode kernel of their own; a row costs a 32-row tile
# there, so many of them are better off in the decode kernel, which takes a group's heads as its columns.
SINGLE_ROWS_RIDE_ALONG = 128
PREFILL_MAX_CACHE_BYTES = 1 << 35      # the prefill attention kernel addresses a cache plane in 32-bit units of 8 bytes


def prefill_addressable(k_cache: torch.Tensor) -> bool:
    """Whether the prefill attention kernel can address this cache plane: under 32 GB, pages under 128 MB, under 2^24 pages."""
    pages, page_bytes = k_cache.shape[0], k_cache[0].numel() * k_cache.element_size()
    return pages * page_bytes < PREFILL_MAX_CACHE_BYTES and page_bytes < (1 << 27) and pages < (1 << 24)


def mfma_block_size(block_size: int) -> bool:
    """Block sizes the matrix-core attention kernels take: powers of two from 4 (others go to the generic kernel)."""
    return block_size >= 4 and block_size & (block_size - 1) == 0


def decode_splits(num_seqs: int, num_kv_heads: int, max_context: int, block_size: int = 16) -> int:
    """How many ways the keys of each sequence are split so that a decode step fills the GPU.

    Never more than ``MAX_KEY_SPLITS``, which is what the kernel and its merge take. With pages of 16
    positions or more the kernel keeps several tiles of keys in flight a wave, a wave is a workgroup, and the
    GPU holds 1024 of them at a time, four a compute unit. About 512 waves with shares of at least 128 keys
    measured best from batch 1 to 128 where that many waves spread evenly; where they do not (24 sequences of 8
    KV heads in 3 shares are 576 waves: two compute units in three carry two, the others three) up to twice the
    shares are tried for the count that leaves the fewest compute units waiting, each further share weighed at
    1 % for what it writes and the merge reads (batch 24 at 4096 keys: 4 shares, 73.5 against 82.8 µs a layer;
    batch 40: 3 shares, 115 against 125; batch 12: 8 shares, 42 against 48). With exactly 256 (sequence, KV head)
    pairs one wave each walks its whole sequence and nothing is merged (batch 32: 93 against 96 µs). With smaller
    pages a wave has one tile in flight and the GPU wants four times the waves.
    """
    if block_size >= 16:
        pairs = max(1, num_seqs * num_kv_heads)
        if pairs == 256:
            return 1
        by_length = max(1, max_context // 128)          # at least four 32-key tiles a share
        most = min(by_length, MAX_KEY_SPLITS)
        first = -(-512 // pairs)
        if first >= most:
            return max(1, most)
        best, best_cost = first, None
        for n in range(first, min(2 * first, most) + 1):
            waves = pairs * n
            if n > first and waves > 1024:
                break
            cost = -(-waves // 256) * 256 / waves * (1 + 0.01 * n)
            if best_cost is None or cost < best_cost:
                best, best_cost = n, cost
        return best
    by_occupancy = -(-2048 // max(1, num_seqs * num_kv_heads))     # about 2048 waves ...
    if by_occupancy > 16:
        by_occupancy = -(-by_occupancy // 2)        # ... but half as many where that still leaves many shares to merge
    by_length = max(1, max_context // 64)           # at least two 32-key tiles a share
    return max(1, min(by_occupancy, by_length, MAX_KEY_SPLITS))


# Shares of one length for all sequences (``decode_share_plan``): the grid holds at least this many a sequence.
BALANCED_SHARES_GRID = 8
# Where each sequence's own shares would be this few at most, shares of one length are taken if they halve the
# longest share; with more shares of its own a sequence's waves are short already, and only a share four times
# shorter pays (16 sequences of 8 KV heads, 100 to 4000 keys, 4 shares each: 37.7 us a layer, shares of one
# length 36.8 to 44.8; one sequence of 32 k keys beside 23 of 1 k: 176 -> 74).
BALANCED_SHARES_MAX_EQUAL = 3


def decode_share_plan(context_lens, num_kv_heads: int, plan_context: int, block_size: int = 16,
                      window: Optional[int] = None) -> "tuple":
    """``(shares, share_tiles)`` for a step of single decoded tokens over sequences of these lengths.

    ``share_tiles`` = 0: every sequence's keys go into ``shares`` equal parts of its own (``decode_splits``): the
    rule for sequences of about one length. A wave walks its share tile after tile, so the longest share sets
    the kernel's time, and with sequences of very different lengths (the longest a quarter above the mean) that
    is the longest sequence's, while the waves of the short ones are done early (32 sequences of 8 KV heads, 65 k
    keys in all: 51 us a layer with 2048 each, 79 with 100 to 4000, 87 with a quarter of them 4096 long; 2 of 4096
    beside 30 of 600: 83 for 26 k keys; one of 32 k beside 7 of 1 k: 89, as much as half of 8 of 32 k). Then all
    shares get ONE length, ``share_tiles`` tiles of 32 keys: the smallest for which the waves that have keys at all
    stay within 512 (768 above 128 (sequence, KV head) pairs, 1024 above 256). A short sequence fills one share, a long one many,
    and the rest of the grid (a power of two of shares a sequence, so that a recorded step serves while the lengths
    grow) is empty (those steps: 68, 62, 43 and 52 us; 64 sequences, 2 of them long: 94 -> 53). Taken only if the
    longest share gets half as long, a quarter where a sequence's own shares are more than three: between that
    and equal the merge and the empty shares cost what the balance gains (56 sequences, a quarter long: 94 -> 109
    us at two thirds; two of 16 k beside six of 2 k: 56 -> 57 at a third).
    """
    S = len(context_lens)
    equal = decode_splits(S, num_kv_heads, plan_context, block_size)
    if block_size < 16 or S < 2 or BALANCED_SHARES_MAX_EQUAL <= 0:
        return equal, 0
    tiles = []
    for n in context_lens:
        pos = n - 1
        first = max(0, pos - window + 1) // 32 if window else 0
        tiles.append(pos // 32 + 1 - first)
    longest = max(tiles)
    if longest * S < 1.25 * sum(tiles):
        return equal, 0
    pairs = S * num_kv_heads
    target = (512 if pairs <= 128 else 768 if pairs <= 256 else 1024) // num_kv_heads      # waves with keys, a KV head
    if target <= S:
        return equal, 0
    lo, hi = max(4, -(-longest // MAX_KEY_SPLITS)), longest      # a share of at least 128 keys, the longest within the grid
    while lo < hi:                                               # the count of waves falls as the shares grow
        mid = (lo + hi) // 2
        if sum(-(-t // mid) for t in tiles) <= target:
            hi = mid
        else:
            lo = mid + 1
    before = -(-longest // equal)
    if (2 * lo > before) if equal <= BALANCED_SHARES_MAX_EQUAL else (4 * lo >= before):
        return equal, 0
    grid = BALANCED_SHARES_GRID
    while grid * lo < longest:
        grid *= 2
    return grid, lo


def step_key_shares(step, num_seqs: int, num_kv_heads: int, plan_context: int, block_size: int) -> "tuple":
    """``(shares, share_tiles tensor or None)`` of a decode step: what the step's builder planned for this cache
    group (``key_shares`` of the group's view of the step), else the rule by the step's size alone."""
    planned = getattr(step, "key_shares", None)
    if planned is not None:
        return planned
    return decode_splits(num_seqs, num_kv_heads, plan_context, block_size), None


def check_attention_sizes(num_heads: int, num_kv_heads: int, head_dim: int) -> None:
    """Refuses, when a model is built, head geometries that no attention kernel here takes."""
    if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
        raise InvalidArgument(f"{num_heads} query heads are not a positive multiple of {num_kv_heads} kv heads")
    if head_dim <= 0 or head_dim % 2 or head_dim > MAX_HEAD_DIM:
        raise InvalidArgument(f"head_dim {head_dim} must be even and at most {MAX_HEAD_DIM}: no attention kernel of "
                              f"this engine takes it")


def attention_decode_bf16(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                          query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                          num_seqs: int, num_heads: int, scale: float, window: Optional[int], nsplit: int,
                          part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                          seq_ids: Optional[torch.Tensor] = None, depth: int = 0,
                          share_tiles: Optional[torch.Tensor] = None, softcap: Optional[float] = None,
                          chunk: Optional[int] = None, sinks: Optional[torch.Tensor] = None,
                          keep_first: int = 0) -> None:
    """Attention for sequences that bring one new row each (``seq_ids`` selects them; None = all).

    ``chunk`` n (instead of a ``window``): a query at position p reads the keys from ``p - p % n`` on. ``sinks``
    (float32 ``[heads]``): ``exp(sinks[h])`` is one more term of head h's softmax denominator. ``keep_first`` f
    (beside a ``window``, with uncapped scores): the keys of positions below f are read as well.

    ``share_tiles`` (one int32 on the device, or None): the length of every share in tiles of 32 keys, for steps
    whose sequences differ much in length (``decode_share_plan``); with pages of 16 positions or more and more than
    one share.

    ``depth`` picks the kernel (0: by the library's rule; 1: page lookups per lane, any page size; 2 to 4: that
    many tiles of keys in registers, pages of 16 positions or more); all give the same bits.
    """
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H = num_heads
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise InvalidArgument("attention_decode_bf16 takes bfloat16 queries, cache and output")
    if q.shape[1] != H * Dh or out.shape != q.shape:
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if Dh not in MFMA_HEAD_DIMS or H % KVH or not mfma_block_size(bs):
        raise InvalidArgument(f"attention_decode_bf16 takes head sizes in steps of 16 up to 256 and block sizes 4, 8, "
                              f"16, ...; got head_dim {Dh}, {H}/{KVH} heads, block {bs}")
    _i32(query_start, "query_start")
    _i32(context_lens, "context_lens")
    _i32(block_tables, "block tables")
    if seq_ids is not None:
        _i32(seq_ids, "sequence ids", num_seqs)
    if not 1 <= nsplit <= MAX_KEY_SPLITS:
        raise InvalidArgument(f"attention_decode_bf16 cuts the keys into 1 to {MAX_KEY_SPLITS} shares, got {nsplit}")
    if nsplit > 1:
        _f32(part_o, "split accumulators")
        _f32(part_ml, "split maxima and sums")
        if part_o.numel() < num_seqs * H * nsplit * Dh or part_ml.numel() < num_seqs * H * nsplit * 2:
            raise InvalidArgument("the buffers for the splits are too small")
    lib = _lib("attention_decode_bf16", Dh)
    if not 0 <= depth <= 4 or (depth > 1 and bs < 16):
        raise InvalidArgument(f"attention_decode_bf16: depth {depth} with pages of {bs} positions")
    if share_tiles is not None:
        _i32(share_tiles, "the shares' length", 1)
        if nsplit == 1 or bs < 16 or depth == 1:
            raise InvalidArgument("a length for all shares goes with more than one share and pages of 16 positions or more")
    if keep_first and (not window or softcap):
        raise InvalidArgument("first positions are kept beside a sliding window, with uncapped scores")
    _call(lib.tie_attention_decode_bf16_keeping, "attention_decode_bf16",
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(part_o), _ptr(part_ml),
        query_start.data_ptr(), context_lens.data_ptr(), block_tables.data_ptr(), _ptr(seq_ids), num_seqs, H, KVH, bs,
        block_tables.shape[1], float(scale), float(softcap or 0.0), int(window or 0), nsplit, _ptr(share_tiles), depth,
        int(chunk or 0), _ptr(_sinks(sinks, H, window, chunk)), int(keep_first or 0), _stream())


def _sinks(sinks: Optional[torch.Tensor], heads: int, window, chunk) -> Optional[torch.Tensor]:
    if window and chunk:
        raise InvalidArgument("attention takes a sliding window or causal chunks, not both")
    return None if sinks is None else _f32(sinks, "attention sinks", (heads,))


def decode_attention_prepares(batch, q_dtype: torch.dtype, k_cache: torch.Tensor, num_heads: int) -> bool:
    """Whether a step runs on the decode attention kernel that makes its own queries, newest keys and values
    from the QKV projection's planes: single decoded tokens only, bfloat16, pages of 16 positions or more,
    head sizes 32, 64, 128 or 256, at most 16 query heads a KV head, fewer than 512 (sequence, KV head) pairs."""
    NB, KVH, bs, Dh = k_cache.shape
    if not (batch.all_decode and q_dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16
            and Dh in (32, 64, 128, 256) and bs >= 16 and mfma_block_size(bs)
            and num_heads % KVH == 0 and num_heads // KVH <= 16):
        return False
    # With so many sequences that the keys are not cut into shares, every wave would make a newest key and value
    # and attend to it after its tiles, and the step is a little slower that way than with the q/k kernel before
    # it (batch 64 at the 8B shape: 0.7 %).
    return batch.num_seqs * KVH < 512


def paged_attention_prepared(planes: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                             eps: float, angles: torch.Tensor, write_kv: bool, k_cache: torch.Tensor,
                             v_cache: torch.Tensor, out: torch.Tensor, step, batch, num_heads: int, scale: float,
                             window: Optional[int], scratch) -> None:
    """Attention of a step of single decoded tokens straight from the QKV projection's planes of partial sums
    (``planes`` float32 ``[P, rows, (H + 2 KVH) * Dh]``): the kernel sums the planes, applies the per-head
    RMS norm (weights or None) and the rotation by ``angles`` (``[rows, Dh]``: cos, then sin), writes the newest
    key and value into the cache (unless ``write_kv`` is false) and attends; see ``decode_attention_prepares``."""
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H, S = num_heads, batch.num_seqs
    if not decode_attention_prepares(batch, out.dtype, k_cache, H):
        raise InvalidArgument("this step does not run on the decode attention kernel that prepares its own queries")
    _f32(planes, "QKV planes")
    _f32(angles, "rotation angles")
    _gpu(out, "attention output")
    P, rows, width = planes.shape
    if not planes.is_contiguous() or width < (H + 2 * KVH) * Dh or rows != out.shape[0] or out.shape[1] != H * Dh:
        raise InvalidArgument(f"QKV planes {list(planes.shape)} / out {list(out.shape)} do not fit {H} + 2 x {KVH} heads of {Dh}")
    if angles.shape != (rows, Dh) or not angles.is_contiguous() or not 1 <= P <= 8:
        raise InvalidArgument(f"angles {list(angles.shape)} for {rows} rows of head_dim {Dh}, {P} planes")
    for w, name in ((q_weight, "q norm weight"), (k_weight, "k norm weight")):
        if w is not None:
            _f32(w, name, (Dh,))
    nsplit, share_tiles = step_key_shares(step, S, KVH, batch.plan_context, bs)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = scratch("attention.split_o", (S * H * nsplit * Dh,), torch.float32)
        part_ml = scratch("attention.split_ml", (S * H * nsplit * 2,), torch.float32)
    _call(_lib("attention_decode_bf16", Dh).tie_attention_decode_prepared_bf16, "attention_decode_prepared_bf16",
          planes.data_ptr(), rows * width, P, width, _ptr(q_weight), _ptr(k_weight), float(eps), angles.data_ptr(),
          int(bool(write_kv)), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(part_o), _ptr(part_ml),
          batch.query_start.data_ptr(), batch.context_lens.data_ptr(), step.block_tables.data_ptr(), None, S, H, KVH,
          bs, step.block_tables.shape[1], float(scale), int(window or 0), nsplit, _ptr(share_tiles), 0, _stream())


def prefill_items(new_tokens, group_size: int) -> "list":
    """Work items ``(sequence, first new row)`` of the prefill attention kernel for one step.

    An item is one workgroup: 32, 64 or 128 consecutive new rows of a sequence, depending on how
    many query heads share a KV head (four (head, 32-row tile) pairs run side by side).
    """
    heads_at_once = min(group_size, 4)
    rows = 32 * (1 if heads_at_once >= 3 else 4 // heads_at_once)
    items = []
    for s, n in enumerate(new_tokens):
        for first in range(0, n, rows):
            items.append((s, first))
    return items


def prefill_loads_straight(head_dim: int, block_size: int) -> bool:
    """Whether the prefill attention kernel that loads its tiles straight into LDS takes this geometry
    (it has no limit on the cache's size: its addresses are 64-bit scalars)."""
    return head_dim in (32, 64, 128, 256) and block_size >= 16 and mfma_block_size(block_size)


def attention_prefill_bf16(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                           query_start: torch.Tensor, context_lens: torch.Tensor, block_tables: torch.Tensor,
                           items: torch.Tensor, num_heads: int, scale: float, window: Optional[int] = None,
                           nsplit: int = 1, part_o: Optional[torch.Tensor] = None,
                           part_ml: Optional[torch.Tensor] = None, merge_rows: Optional[torch.Tensor] = None,
                           staging: int = 0, softcap: Optional[float] = None, chunk: Optional[int] = None,
                           sinks: Optional[torch.Tensor] = None, keep_first: int = 0) -> None:
    """Causal attention of the new rows of the sequences ``items`` names over their cached keys.

    ``keep_first`` f (beside a ``window``, with uncapped scores): the keys of positions below f are read as well;
    such steps copy their tiles through registers.

    ``staging`` picks how key tiles reach LDS: 1 = copied through registers (any page and head size),
    2 = loaded straight into LDS (``prefill_loads_straight``), 0 = the second where it applies.

    ``nsplit`` > 1 cuts every item's keys into that many shares (one workgroup each) for steps with few
    items and long contexts; ``part_o`` / ``part_ml`` (float32, ``rows * H * nsplit * Dh`` and ``* 2``
    with rows = all rows of the step) take the partial results and ``merge_rows`` lists the rows
    that the items cover, which a second kernel then merges.
    """
    _gpu(q, "queries")
    _gpu(out, "attention output")
    _gpu(k_cache, "k cache")
    _gpu(v_cache, "v cache")
    NB, KVH, bs, Dh = k_cache.shape
    _check_cache(k_cache, v_cache, KVH, bs, Dh)
    H = num_heads
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise InvalidArgument("attention_prefill_bf16 takes bfloat16 queries, cache and output")
    if q.shape[1] != H * Dh or out.shape != q.shape:
        raise InvalidArgument(f"attention: q {list(q.shape)} / out {list(out.shape)} do not fit {H} heads of {Dh}")
    if Dh not in MFMA_HEAD_DIMS or H % KVH or not mfma_block_size(bs):
        raise InvalidArgument(f"attention_prefill_bf16 takes head sizes in steps of 16 up to 256 and block sizes 4, 8, "
                              f"16, ...; got head_dim {Dh}, {H}/{KVH} heads, block {bs}")
    if staging not in (0, 1, 2) or (staging == 2 and not prefill_loads_straight(Dh, bs)):
        raise InvalidArgument(f"attention_prefill_bf16: staging {staging} with head_dim {Dh} and pages of {bs} positions")
    if keep_first and (not window or softcap or staging == 2):
        raise InvalidArgument("first positions are kept beside a sliding window, with uncapped scores and tiles copied "
                              "through registers")
    if staging == 0:
        staging = 2 if prefill_loads_straight(Dh, bs) and not keep_first else 1
    if staging == 1 and not prefill_addressable(k_cache):
        raise InvalidArgument(f"attention_prefill_bf16 addresses cache planes under 32 GB (pages under 128 MB, under 2^24 "
                              f"pages); got {NB} pages of {k_cache[0].numel() * k_cache.element_size()} bytes")
    _i32(query_start, "query_start")
    _i32(context_lens, "context_lens")
    _i32(block_tables, "block tables")
    _i32(items, "work items")
    if items.dim() != 2 or items.shape[1] != 2 or items.shape[0] == 0:
        raise InvalidArgument("work items must be a non-empty [n, 2] tensor")
    num_merge = 0
    if nsplit > 1:
        _f32(part_o, "split accumulators")
        _f32(part_ml, "split maxima and sums")
        _i32(merge_rows, "rows to merge")
        rows = q.shape[0]
        num_merge = merge_rows.numel()
        if part_o.numel() < rows * H * nsplit * Dh or part_ml.numel() < rows * H * nsplit * 2 or not 0 < num_merge <= 65535:
            raise InvalidArgument("the buffers for the splits are too small, or no (or too many) rows to merge")
    lib = _lib("attention_prefill_bf16", Dh)
    _call(lib.tie_attention_prefill_bf16_keeping, "attention_prefill_bf16",
        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), query_start.data_ptr(),
        context_lens.data_ptr(), block_tables.data_ptr(), items.data_ptr(), items.shape[0], H, KVH, bs,
        block_tables.shape[1], float(scale), float(softcap or 0.0), int(window or 0), int(nsplit), _ptr(part_o),
        _ptr(part_ml), _ptr(merge_rows), num_merge, staging, int(chunk or 0),
        _ptr(_sinks(sinks, num_heads, window, chunk)), int(keep_first or 0), _stream())


def prefill_splits(num_items: int, num_kv_heads: int, group_size: int, max_context: int, num_rows: int) -> int:
    """Shares the keys of every prefill item are cut into: more than one only where the items alone leave CUs idle."""
    passes = -(-group_size // min(group_size, 4))
    workgroups = num_items * num_kv_heads * passes
    if workgroups >= 256 or num_rows > 65535:
        return 1
    by_fill = 512 // max(1, workgroups)
    by_length = max(1, -(-max_context // 64) // 4)          # at least four 64-key tiles a share
    return max(1, min(8, by_fill, by_length))


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, step, batch,
                    num_heads: int, scale: float, window: Optional[int] = None, scratch=None,
                    softcap: Optional[float] = None, chunk: Optional[int] = None,
                    sinks: Optional[torch.Tensor] = None, keep_first: int = 0) -> None:
    """Causal attention over the paged cache for one step's batch, on the fastest kernel that takes it.

    ``step`` is the cache group's view of the step (block tables), ``batch`` the step's arrays
    (query_start, context_lens, seq_of_row) and host-side numbers; ``scratch(name, shape, dtype)``
    hands out workspace for the partial results of split keys.
    """
    NB, KVH, bs, Dh = k_cache.shape
    fast = (q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and Dh in MFMA_HEAD_DIMS
            and num_heads % KVH == 0 and mfma_block_size(bs) and scratch is not None)
    if keep_first and not window:
        raise InvalidArgument("first positions are kept beside a sliding window only")
    if keep_first and softcap:
        fast = False           # kept first positions beside capped scores: the generic kernel alone takes both
    reach = (window + keep_first if window else None) or chunk      # the most keys a query reads: what the shares of a sequence's keys are planned by
    if fast and batch.all_decode:          # more than 16 query heads a KV head: several waves of 16 columns
        S = batch.num_seqs
        nsplit, share_tiles = step_key_shares(step, S, KVH, batch.plan_context, bs)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = scratch("attention.split_o", (S * num_heads * nsplit * Dh,), torch.float32)
            part_ml = scratch("attention.split_ml", (S * num_heads * nsplit * 2,), torch.float32)
        attention_decode_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                              S, num_heads, scale, window, nsplit, part_o, part_ml, share_tiles=share_tiles,
                              softcap=softcap, chunk=chunk, sinks=sinks, keep_first=keep_first)
        return
    if fast:
        # A mixed step: sequences that bring one decoded token go to the decode kernel (their keys are
        # split over many waves), the prompt portions to the prefill kernel. Built once a step.
        G = num_heads // KVH
        key = ("attention_work", G)
        work = batch.memo.get(key)
        if work is None:
            new = batch.host_new_tokens
            single = [s for s, n in enumerate(new) if n == 1]
            if len(single) == len(new):
                single = []                                   # nothing but single rows and yet not a decode step
            elif len(single) * KVH * -(-G // min(G, 4)) <= SINGLE_ROWS_RIDE_ALONG:
                single = []         # a few single rows: items of the prefill kernel, one launch and one merge less
            taken = set(single)
            items = [it for it in prefill_items(new, G) if it[0] not in taken]
            starts = [0]
            for n in new:
                starts.append(starts[-1] + n)
            merge_rows = [starts[s] + r for s in sorted({it[0] for it in items}) for r in range(new[s])]
            work = batch.memo[key] = (
                torch.tensor(single, dtype=torch.int32).to(q.device) if single else None, len(single),
                torch.tensor(items, dtype=torch.int32).to(q.device) if items else None, len(items),
                torch.tensor(merge_rows, dtype=torch.int32).to(q.device) if items else None,
                max((batch.host_context_lens[it[0]] for it in items), default=0))
        seq_ids, num_single, items, num_items, merge_rows, items_context = work
        if num_single:
            shares_key = ("single_row_shares", KVH, reach)
            planned = batch.memo.get(shares_key)
            if planned is None:                # this step runs eagerly: the shares' length goes to the device by itself
                lens = [c for c, n in zip(batch.host_context_lens, batch.host_new_tokens) if n == 1]
                nsplit, length = decode_share_plan(lens, KVH, batch.plan_context, bs, reach)
                planned = batch.memo[shares_key] = (
                    nsplit, torch.tensor([length], dtype=torch.int32).to(q.device) if length else None)
            nsplit, share_tiles = planned
            part_o = part_ml = None
            if nsplit > 1:
                part_o = scratch("attention.split_o", (num_single * num_heads * nsplit * Dh,), torch.float32)
                part_ml = scratch("attention.split_ml", (num_single * num_heads * nsplit * 2,), torch.float32)
            attention_decode_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                                  num_single, num_heads, scale, window, nsplit, part_o, part_ml, seq_ids=seq_ids,
                                  share_tiles=share_tiles, softcap=softcap, chunk=chunk, sinks=sinks,
                                  keep_first=keep_first)
        if items is not None and (keep_first or not prefill_loads_straight(Dh, bs)) and not prefill_addressable(k_cache):
            # A cache plane the prefill kernel cannot address: the prompt portions go to the generic kernel
            # (which runs every row of the step; the single rows above are simply computed again).
            paged_attention_generic(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                                    batch.seq_of_row, num_heads, scale, window, softcap, chunk, sinks, keep_first)
            return
        if items is not None:
            rows = q.shape[0]
            # by the longest context among the portions themselves: a single row of 32 k keys beside them says nothing
            # about how many tiles a portion's share would hold
            nsplit = prefill_splits(num_items, KVH, G, items_context, rows)
            part_o = part_ml = None
            if nsplit > 1:
                part_o = scratch("attention.prefill_split_o", (rows * num_heads * nsplit * Dh,), torch.float32)
                part_ml = scratch("attention.prefill_split_ml", (rows * num_heads * nsplit * 2,), torch.float32)
            attention_prefill_bf16(q, k_cache, v_cache, out, batch.query_start, batch.context_lens,
                                   step.block_tables, items, num_heads, scale, window, nsplit, part_o, part_ml,
                                   merge_rows if nsplit > 1 else None, softcap=softcap, chunk=chunk, sinks=sinks,
                                   keep_first=keep_first)
        return
    paged_attention_generic(q, k_cache, v_cache, out, batch.query_start, batch.context_lens, step.block_tables,
                            batch.seq_of_row, num_heads, scale, window, softcap, chunk, sinks, keep_first)


# ------------------------------------------------------------------ mixers with a state of fixed size
DECAY_ATTENTION_MAX_DIM = 512      # rows of a head's state the scan kernel keeps in registers (a quarter of them a wave)
SCAN_CHUNK_ROWS = 64               # rows of a chunk where a long portion's recurrence runs chunk beside chunk
SCAN_CHUNKS_FROM = 128             # a step's longest portion from which the recurrences run in chunks


class ScanChunks:
    """A step's rows cut into chunks for the recurrences: ``items`` int32 ``[count, 3]`` = (sequence, first row, one
    past the last row) in the order of the rows, ``first_item`` int32 ``[S + 1]`` the sequences' ranges of items."""

    def __init__(self, items: torch.Tensor, first_item: torch.Tensor, count: int, longest: int = 0):
        self.items, self.first_item, self.count = items, first_item, count
        self.longest = longest            # rows of the longest chunk


def scan_chunks(batch, device, rows: int = SCAN_CHUNK_ROWS, force: bool = False) -> Optional[ScanChunks]:
    """The chunks of a step with a long portion (None for steps of short ones: each sequence then runs in one go).
    Built once a step from the host-side counts - steps with prompt portions are never recorded - and shared by
    all layers through ``batch.memo``."""
    new = batch.host_new_tokens
    if not force and max(new) < SCAN_CHUNKS_FROM:
        return None
    key = ("scan_chunks", rows)
    memo = batch.memo.get(key)
    if memo is None:
        items, first, row = [], [0], 0
        for s, n in enumerate(new):
            pieces = -(-n // rows)
            for i in range(pieces):              # pieces of nearly one length
                a, b = row + n * i // pieces, row + n * (i + 1) // pieces
                items.append((s, a, b))
            row += n
            first.append(len(items))
        if len(items) > MAX_STEP_TOKENS:
            return None
        memo = batch.memo[key] = ScanChunks(torch.tensor(items, dtype=torch.int32).to(device),
                                            torch.tensor(first, dtype=torch.int32).to(device), len(items),
                                            max(b - a for _, a, b in items))
    return memo


def decay_attention_scan(proj: torch.Tensor, out: torch.Tensor, state: torch.Tensor, query_start: torch.Tensor,
                         state_slots: torch.Tensor, decay: torch.Tensor, num_seqs: int, heads: int, key_dim: int,
                         value_dim: int, activation: str = "silu", chunks: Optional[ScanChunks] = None,
                         scratch=None) -> None:
    """Linear attention with a decay per head, token by token through each sequence's state.

    ``S_t = decay[h] * S_(t-1) + k_t v_t^T``, ``out_t = S_t^T q_t`` with ``q, k, v = act(proj columns)``; ``proj``
    float32 rows ``[q (heads * key_dim) | k (heads * key_dim) | v (heads * value_dim) | ...]``; ``state`` float32
    ``[slots, heads, key_dim, value_dim]``, read at and written back to ``state_slots[s]`` for the rows
    ``query_start[s] .. query_start[s + 1] - 1`` of every sequence s. ``out`` float32 ``[T, heads * value_dim]``.

    With ``chunks`` (``scan_chunks``; ``scratch(name, shape, dtype)`` hands out the memory for the chunks' states)
    the rows run chunk beside chunk in three launches: every chunk from zero, the chunks' states combined in
    order, every chunk again from its true start. The same values up to rounding."""
    _gpu_strided(proj, "projection rows")
    if proj.dtype != torch.float32:
        raise InvalidArgument(f"projection rows must be float32, got {proj.dtype}")
    T = proj.shape[0]
    _f32(out, "linear attention output", (T, heads * value_dim))
    _f32(state, "linear attention state")
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, key_dim, value_dim):
        raise InvalidArgument(f"state {list(state.shape)} does not fit {heads} heads of {key_dim} x {value_dim}")
    if key_dim > DECAY_ATTENTION_MAX_DIM:
        raise InvalidArgument(f"a key size of {key_dim} exceeds the {DECAY_ATTENTION_MAX_DIM} this kernel takes")
    if proj.shape[1] < heads * (2 * key_dim + value_dim):
        raise InvalidArgument(f"projection rows hold {proj.shape[1]} values, {heads * (2 * key_dim + value_dim)} are needed")
    if activation not in ("silu", "none"):
        raise InvalidArgument(f"activation '{activation}' (supported: silu, none)")
    _i32(query_start, "query_start", num_seqs + 1)
    _i32(state_slots, "state slots", num_seqs)
    _f32(decay, "decay", (heads,))
    chunk_states = None
    if chunks is not None:
        chunk_states = scratch("scan.chunk_states", (chunks.count, heads, key_dim, value_dim), torch.float32)
    _call(_lib("recurrent").tie_decay_attention_scan, "decay_attention_scan", proj.data_ptr(), proj.stride(0),
          out.data_ptr(), state.data_ptr(), query_start.data_ptr(), state_slots.data_ptr(), decay.data_ptr(),
          num_seqs, heads, key_dim, value_dim, int(activation == "silu"),
          _ptr(chunks.items) if chunks else None, _ptr(chunks.first_item) if chunks else None,
          chunks.count if chunks else 0, _ptr(chunk_states), chunks.longest if chunks else 0, _stream())


def gated_rms_norm(o: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor, out: torch.Tensor) -> None:
    """out = RMSNorm(o) * weight * sigmoid(gate) row by row; ``o`` float32 ``[T, n]``, ``gate`` float32 rows of n
    (a view whose rows may lie further apart), ``out`` float32 or bfloat16."""
    _f32(o, "gated norm input")
    T, n = o.shape
    _f32(weight, "gated norm weight", (n,))
    _gpu_strided(gate, "gate rows")
    if gate.dtype != torch.float32 or tuple(gate.shape) != (T, n):
        raise InvalidArgument(f"gate rows {list(gate.shape)} {gate.dtype} do not fit float32 {[T, n]}")
    _gpu(out, "gated norm output")
    if tuple(out.shape) != (T, n):
        raise InvalidArgument(f"gated norm output {list(out.shape)} does not match input {[T, n]}")
    _call(_lib("recurrent").tie_gated_rms_norm, "gated_rms_norm", o.data_ptr(), weight.data_ptr(), float(eps),
          gate.data_ptr(), gate.stride(0), out.data_ptr(), _code(out, "gated norm output"), T, n, _stream())


def min_gru_scan(proj: torch.Tensor, out: torch.Tensor, state: torch.Tensor, query_start: torch.Tensor,
                 state_slots: torch.Tensor, num_seqs: int, width: int, chunks: Optional[ScanChunks] = None,
                 scratch=None, bias: Optional[torch.Tensor] = None) -> None:
    """The minimal gated recurrent unit, element by element, token by token through each sequence's state.

    ``proj`` float32 rows ``[a | u | g]`` of ``width`` each, to which ``bias`` (float32 ``[3 * width]``, or None)
    is added as they are read: ``z = sigmoid(a)``, candidate
    ``u + 1/2`` for ``u >= 0`` and ``sigmoid(u)`` below, ``S_t = (1 - z) S_(t-1) + z * candidate``,
    ``out_t = S_t * silu(g)``. ``state`` float32 ``[slots, width]``; ``out`` float32 or bfloat16 ``[T, width]``.
    ``chunks`` and ``scratch`` as for ``decay_attention_scan``."""
    _gpu_strided(proj, "projection rows")
    if proj.dtype != torch.float32 or proj.shape[1] < 3 * width:
        raise InvalidArgument(f"projection rows {list(proj.shape)} {proj.dtype} do not hold three float32 runs of {width}")
    T = proj.shape[0]
    _gpu(out, "recurrence output")
    if tuple(out.shape) != (T, width):
        raise InvalidArgument(f"recurrence output {list(out.shape)} does not fit {[T, width]}")
    _f32(state, "recurrence state")
    if state.dim() != 2 or state.shape[1] != width:
        raise InvalidArgument(f"state {list(state.shape)} does not fit a width of {width}")
    _i32(query_start, "query_start", num_seqs + 1)
    _i32(state_slots, "state slots", num_seqs)
    chunk_ab = scratch("scan.chunk_ab", (2, chunks.count, width), torch.float32) if chunks is not None else None
    _call(_lib("recurrent").tie_min_gru_scan, "min_gru_scan", proj.data_ptr(), proj.stride(0), out.data_ptr(),
          _code(out, "recurrence output"), state.data_ptr(), query_start.data_ptr(), state_slots.data_ptr(),
          num_seqs, width, _ptr(chunks.items) if chunks else None, _ptr(chunks.first_item) if chunks else None,
          chunks.count if chunks else 0, _ptr(chunk_ab),
          _ptr(_f32(bias, "recurrence bias", (3 * width,)) if bias is not None else None), _stream())


# ------------------------------------------------------- routed feed-forward (mixture of experts)
MOE_MAX_EXPERTS = 1024       # MOE_MAX_EXPERTS of csrc/moe.hip


MOE_MAX_GROUP_TOP = 8         # MOE_MAX_GROUP_TOP of csrc/moe.hip


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], groups: int, keep: int, top: int,
              ids: torch.Tensor, weights: torch.Tensor, scoring: str = "softmax", group_top: int = 1,
              renormalize: bool = False, renorm_eps: float = 0.0, weight_scale: float = 1.0, shared: int = 0) -> None:
    """The router's choice for every row of float32 ``logits [T, E]`` (``[T, E + 1]`` with ``shared``).

    ``s = softmax(logits)`` over the experts, or with ``scoring`` ``"sigmoid"`` ``sigmoid(logits)`` expert by expert;
    the choice looks at ``s + correction``: the experts form ``groups`` equal groups of neighbours, a group scores
    the sum of its ``group_top`` best members (1: its best member), only members of the ``keep`` best groups stay
    eligible, and the ``top`` best of those are chosen (ties to the lower index) into ``ids`` int32; ``weights``
    float32 are ``s`` at the chosen, with ``renormalize`` divided by their sum + ``renorm_eps``, times
    ``weight_scale``. ``shared`` n: both arrays are ``[T, top + n]``, the last n slots of a row name the experts
    ``E .. E + n - 1`` (experts every row uses) with the weight ``sigmoid(logits[:, E])``.
    """
    _f32(logits, "router logits")
    T, row = logits.shape
    E = row - (1 if shared else 0)
    slots = top + shared
    if correction is not None:
        _f32(correction, "the choice's correction", (E,))
    _i32(ids, "chosen experts")
    _f32(weights, "routing weights", (T, slots))
    if tuple(ids.shape) != (T, slots):
        raise InvalidArgument(f"chosen experts {list(ids.shape)} do not fit {[T, slots]}")
    if scoring not in ("softmax", "sigmoid"):
        raise InvalidArgument(f"router scoring '{scoring}' (supported: softmax, sigmoid)")
    if not 0 < E <= MOE_MAX_EXPERTS or groups <= 0 or E % groups or not 0 < keep <= groups or not 0 < top <= E or \
            not 0 < group_top <= MOE_MAX_GROUP_TOP or shared < 0:
        raise InvalidArgument(f"moe_route: {E} experts (at most {MOE_MAX_EXPERTS}) in {groups} groups scored by their "
                              f"{group_top} best, {keep} kept, top {top}")
    _call(_lib("moe").tie_moe_route, "moe_route", logits.data_ptr(), row, _ptr(correction), T, E, groups, keep, top,
          int(scoring == "sigmoid"), int(group_top), int(bool(renormalize)), float(renorm_eps), float(weight_scale),
          int(shared), ids.data_ptr(), weights.data_ptr(), _stream())


class ExpertRows:
    """The (row, choice) slots of a step sorted by expert, on the device: see ``moe_align``."""

    __slots__ = ("offsets", "slot_at", "where", "tiles", "num_tiles", "max_tiles", "tile_rows", "slots", "top", "real")


def moe_tile_rows(x_dtype: torch.dtype, w_dtype: torch.dtype, hidden: int, intermediate: int, slots: int,
                  real: int) -> int:
    """Rows of a row tile of the experts' products, which also says which kernels run them: 16, 64 or 128 (by the rows an
    expert gets on average) for the matrix-core kernels, which take bfloat16 rows and weights whose inner sizes
    are multiples of 8; the float32 kernels' tile otherwise."""
    lib = _lib("moe")
    if x_dtype == torch.bfloat16 and w_dtype == torch.bfloat16 and hidden % 8 == 0 and intermediate % 8 == 0:
        return int(lib.tie_moe_bf16_tile_rows(slots, real))
    return int(lib.tie_moe_generic_tile_rows())


def _moe_on_matrix_cores(rows: "ExpertRows", x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gated: bool) -> bool:
    generic = int(_lib("moe").tie_moe_generic_tile_rows())
    if rows.tile_rows == generic:
        return False
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[2] % 8 or \
            out.dtype != (torch.bfloat16 if gated else torch.float32):
        raise InvalidArgument(f"rows sorted in tiles of {rows.tile_rows} go to the matrix-core kernels: bfloat16 rows and "
                              f"weights with an inner size in steps of 8, got {x.dtype}, {w.dtype}, {w.shape[2]}")
    return True


def moe_align(ids: torch.Tensor, real: int, tile_rows: int, scratch) -> ExpertRows:
    """Sorts the slots ``ids [T, top]`` by expert. Choices ``>= real`` name experts without weights: their place is -1.

    ``scratch(name, shape, dtype)`` hands out the int32 arrays: ``offsets [real + 1]``, ``slot_at [slots]``,
    ``where [T, top]``, the row tiles ``[max_tiles, 2]`` (expert, first place) and their number.
    """
    _i32(ids, "chosen experts")
    T, top = ids.shape
    slots = T * top
    if not 0 < real <= MOE_MAX_EXPERTS:
        raise InvalidArgument(f"moe_align takes 1 to {MOE_MAX_EXPERTS} experts, got {real}")
    rows = ExpertRows()
    rows.slots, rows.top, rows.real, rows.tile_rows = slots, top, real, tile_rows
    rows.max_tiles = slots // tile_rows + min(real, slots)
    rows.offsets = scratch("moe.offsets", (real + 1,), torch.int32)
    rows.slot_at = scratch("moe.slot_at", (slots,), torch.int32)
    rows.where = scratch("moe.where", (T, top), torch.int32)
    rows.tiles = scratch("moe.tiles", (rows.max_tiles, 2), torch.int32)
    rows.num_tiles = scratch("moe.num_tiles", (1,), torch.int32)
    _call(_lib("moe").tie_moe_align, "moe_align", ids.data_ptr(), slots, real, tile_rows, rows.offsets.data_ptr(),
          rows.slot_at.data_ptr(), rows.where.data_ptr(), rows.tiles.data_ptr(), rows.max_tiles,
          rows.num_tiles.data_ptr(), _stream())
    return rows


def _moe_weights(w: torch.Tensor, real: int, name: str):
    _gpu(w, name)
    if w.dim() != 3 or w.shape[0] != real:
        raise InvalidArgument(f"{name} must be [{real}, out, in], got {list(w.shape)}")
    return w.shape[1], w.shape[2]


def moe_gate_up(x: torch.Tensor, w_gate: Optional[torch.Tensor], w_up: torch.Tensor, rows: ExpertRows,
                act: torch.Tensor) -> None:
    """``act[place] = silu(x[row] Wg_e^T) * (x[row] Wu_e^T)`` for every sorted slot: ``x [T, K]``, weights
    ``[real, F, K]``. Without gate weights (``w_gate`` None) the experts have no gate and the activation is the square
    of relu: ``act[place] = relu(x[row] Wu_e^T)^2``."""
    _gpu(x, "the experts' input rows")
    _gpu(act, "the experts' activations")
    F_, K = _moe_weights(w_up, rows.real, "up weights")
    mode = 2 if w_gate is None else 1
    if w_gate is not None and (tuple(w_up.shape) != tuple(w_gate.shape) or w_up.dtype != w_gate.dtype or
                               not w_gate.is_contiguous() or not w_gate.is_cuda):
        raise InvalidArgument("gate and up weights must be alike")
    first = w_up if w_gate is None else w_gate
    if x.dim() != 2 or x.shape[1] != K or x.shape[0] * rows.top != rows.slots or tuple(act.shape) != (rows.slots, F_):
        raise InvalidArgument(f"moe_gate_up: rows {list(x.shape)}, activations {list(act.shape)}, weights {list(w_up.shape)}")
    if _moe_on_matrix_cores(rows, x, first, act, True):
        _call(_lib("moe").tie_moe_gemm_bf16, "moe_gate_up", x.data_ptr(), first.data_ptr(),
              w_up.data_ptr() if w_gate is not None else None,
              act.data_ptr(), mode, rows.offsets.data_ptr(), rows.slot_at.data_ptr(), rows.tiles.data_ptr(),
              rows.num_tiles.data_ptr(), rows.max_tiles, rows.tile_rows, rows.top, F_, K, _stream())
        return
    _call(_lib("moe").tie_moe_gemm_generic, "moe_gate_up", x.data_ptr(), _code(x, "rows"), first.data_ptr(),
          w_up.data_ptr() if w_gate is not None else None, _code(first, "expert weights"), act.data_ptr(),
          _code(act, "activations"), mode,
          rows.offsets.data_ptr(), rows.slot_at.data_ptr(), rows.tiles.data_ptr(), rows.num_tiles.data_ptr(),
          rows.max_tiles, rows.top, F_, K, _stream())


def moe_down(act: torch.Tensor, w_down: torch.Tensor, rows: ExpertRows, parts: torch.Tensor) -> None:
    """``parts[place] = act[place] Wd_e^T`` (float32 ``[slots, N]``) for every sorted slot; weights ``[real, N, F]``."""
    _gpu(act, "the experts' activations")
    _f32(parts, "the experts' results")
    N, F_ = _moe_weights(w_down, rows.real, "down weights")
    if tuple(act.shape) != (rows.slots, F_) or tuple(parts.shape) != (rows.slots, N):
        raise InvalidArgument(f"moe_down: activations {list(act.shape)}, results {list(parts.shape)}, weights {list(w_down.shape)}")
    if _moe_on_matrix_cores(rows, act, w_down, parts, False):
        _call(_lib("moe").tie_moe_gemm_bf16, "moe_down", act.data_ptr(), w_down.data_ptr(), None, parts.data_ptr(), 0,
              rows.offsets.data_ptr(), rows.slot_at.data_ptr(), rows.tiles.data_ptr(), rows.num_tiles.data_ptr(),
              rows.max_tiles, rows.tile_rows, rows.top, N, F_, _stream())
        return
    _call(_lib("moe").tie_moe_gemm_generic, "moe_down", act.data_ptr(), _code(act, "activations"), w_down.data_ptr(),
          None, _code(w_down, "down weights"), parts.data_ptr(), F32, 0, rows.offsets.data_ptr(),
          rows.slot_at.data_ptr(), rows.tiles.data_ptr(), rows.num_tiles.data_ptr(), rows.max_tiles, rows.top, N, F_,
          _stream())


def moe_combine(routed: RoutedParts, out: torch.Tensor, accumulate: bool = False) -> None:
    """``out[t] (+)= sum_k weights[t, k] * (parts[where[t, k]] if where[t, k] >= 0 else self_rows[t])``, in the order of k."""
    _f32(out, "the combined result")
    T, n = out.shape
    top = routed.where.shape[1]
    _f32(routed.parts, "the experts' results")
    _i32(routed.where, "places", T * top)
    _f32(routed.weights, "routing weights", (T, top))
    _gpu(routed.self_rows, "input rows")
    if routed.parts.shape[-1] != n or tuple(routed.self_rows.shape) != (T, n):
        raise InvalidArgument("moe_combine: the parts do not fit the result")
    _call(_lib("moe").tie_moe_combine, "moe_combine", routed.parts.data_ptr(), routed.where.data_ptr(),
          routed.weights.data_ptr(), routed.self_rows.data_ptr(), _code(routed.self_rows, "input rows"),
          out.data_ptr(), T, top, n, int(accumulate), _stream())


# ------------------------------------------------- kernels without statistics over a row
def dynamic_tanh(x: torch.Tensor, alpha: Optional[torch.Tensor], weight: Optional[torch.Tensor],
                 bias: Optional[torch.Tensor], out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                 owed: Optional[torch.Tensor] = None) -> None:
    """``out = tanh(alpha * x) * weight + bias`` over rows of the float32 stream ``x`` (``alpha`` a float32 tensor of
    one element, read on the device). ``rows``: gather these rows. ``owed`` (float32 ``[planes, T, n]``): partial sums
    still owed to the stream, added into ``x`` in plane order in the same pass. Without ``alpha`` the function is
    left out: ``out = x`` in the output's type (with the owed sums added)."""
    _f32(x, "the stream")
    _gpu(out, "dynamic_tanh output")
    n = x.shape[-1]
    R = out.numel() // n if n else 0
    if out.shape[-1] != n or (rows is None and x.numel() != out.numel()):
        raise InvalidArgument(f"dynamic_tanh output {list(out.shape)} does not match input {list(x.shape)}")
    plain = alpha is None
    if not plain:
        _f32(alpha, "dynamic_tanh alpha", (1,))
        _f32(weight, "dynamic_tanh weight", (n,))
        _f32(bias, "dynamic_tanh bias", (n,))
    planes = 0
    if owed is not None:
        _f32(owed, "owed partial sums")
        if rows is not None or owed.dim() != 3 or tuple(owed.shape[1:]) != tuple(x.shape):
            raise InvalidArgument(f"owed sums {list(owed.shape)} do not fit the stream {list(x.shape)}")
        planes = owed.shape[0]
    if rows is not None:
        _i32(rows, "dynamic_tanh rows", R)
    if R == 0:
        return
    if R > MAX_STEP_TOKENS:
        raise InvalidArgument(f"a step of {R} rows exceeds the {MAX_STEP_TOKENS} this kernel takes")
    _call(_lib("pointwise").tie_dynamic_tanh, "dynamic_tanh", x.data_ptr(), _ptr(owed), x.numel(), planes,
          _ptr(alpha), _ptr(weight), _ptr(bias), out.data_ptr(), _code(out, "dynamic_tanh output"), _ptr(rows), R, n,
          int(plain), _stream())


def token_gate(gate: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, first: int, out: torch.Tensor) -> None:
    """``out[t, j] = gelu_tanh(gate[t, j]) * table[tokens[t], first + j]``: ``gate`` float32 ``[T, dim]``, ``table``
    ``[vocab, columns]`` (every layer a range of columns of its own), ``out`` ``[T, dim]``."""
    _f32(gate, "the gate's sums")
    _gpu(table, "the per-token table")
    _gpu(out, "gated token rows")
    T, dim = gate.shape
    _i32(tokens, "token ids", T)
    if table.dim() != 2 or first < 0 or first + dim > table.shape[1] or tuple(out.shape) != (T, dim):
        raise InvalidArgument(f"token_gate: table {list(table.shape)}, columns {first} .. {first + dim}, out {list(out.shape)}")
    if T == 0:
        return
    _call(_lib("pointwise").tie_token_gate, "token_gate", gate.data_ptr(), tokens.data_ptr(), table.data_ptr(),
          _code(table, "the per-token table"), table.shape[1], int(first), out.data_ptr(),
          _code(out, "gated token rows"), T, dim, _stream())


# ------------------------------------------------- layer norm, hyper-connections
HYPER_MAX_STREAMS = 8        # HYPER_MAX_STREAMS of csrc/hyper.hip
ROW_IN_LDS_MAX = 16384       # the widest row the kernels that keep a float32 row in LDS take
_NORM_KINDS = {"layer_norm": 0, "rms_norm": 1, None: 2}


def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
               rows: Optional[torch.Tensor] = None) -> None:
    """out = (x - mean) / sqrt(var + eps) * weight row by row (no bias; the variance is the mean of the squared
    deviations; float32 statistics). ``rows`` (int32) picks the rows of ``x`` that are normed."""
    _gpu(x, "layer norm input")
    _gpu(out, "layer norm output")
    n = x.shape[-1]
    count = x.shape[0] if rows is None else rows.numel()
    _f32(weight, "layer norm weight", (n,))
    if x.dim() != 2 or tuple(out.shape) != (count, n) or n > ROW_IN_LDS_MAX:
        raise InvalidArgument(f"layer norm: input {list(x.shape)} / output {list(out.shape)} do not fit {count} rows "
                              f"of at most {ROW_IN_LDS_MAX}")
    if rows is not None:
        _i32(rows, "row indices")
    if count == 0:
        return
    _call(_lib("hyper").tie_layer_norm, "layer_norm", x.data_ptr(), _code(x, "layer norm input"), weight.data_ptr(),
          float(eps), out.data_ptr(), _code(out, "layer norm output"), _ptr(rows), count, n, _stream())


def hyper_connection(streams: torch.Tensor, x: Optional[torch.Tensor] = None, from_x: bool = False, fold: bool = False,
                     write: Optional[tuple] = None, read: Optional[tuple] = None) -> None:
    """One pass over the residual streams ``[S, T, n]`` (float32) of a model with hyper-connections.

    ``write`` ``(y, mix, out)``: every stream t becomes ``sum_s mix[s, t] * stream_s + out[t] * y`` from the old
    streams; ``y`` is float32 rows ``[T, n]`` or planes of partial sums ``[P, T, n]`` added in plane order.
    ``from_x``: the streams do not exist yet; all equal the rows of ``x`` (and are stored). ``fold``: ``x`` receives
    the sum of the (new) streams. ``read`` ``(in, norm_kind, weight, eps, h)``: ``h = norm(sum_s in[s] * stream_s)``
    of the new streams, ``norm_kind`` "layer_norm", "rms_norm" or None (``h`` is then the float32 sum itself)."""
    _f32(streams, "residual streams")
    if streams.dim() != 3 or streams.shape[0] > HYPER_MAX_STREAMS:
        raise InvalidArgument(f"residual streams {list(streams.shape)} must be [streams <= {HYPER_MAX_STREAMS}, rows, width]")
    S, T, n = streams.shape
    if n > ROW_IN_LDS_MAX:
        raise InvalidArgument(f"rows of {n} exceed the {ROW_IN_LDS_MAX} this kernel takes")
    if from_x or fold:
        _f32(x, "the residual rows", (T, n))
    y = mix = out_w = None
    planes, plane_stride = 0, 0
    if write is not None:
        y, mix, out_w = write
        _f32(y, "the sub-layer's result")
        if y.dim() == 2:
            y = y.unsqueeze(0)
        if tuple(y.shape[1:]) != (T, n):
            raise InvalidArgument(f"a sub-layer's result {list(y.shape)} does not fit {T} rows of {n}")
        planes, plane_stride = y.shape[0], y.stride(0)
        _f32(mix, "stream mixing weights", (S, S))
        _f32(out_w, "stream output weights", (S,))
    in_w = w = h = None
    eps, kind, h_code = 0.0, 2, F32
    if read is not None:
        in_w, norm_kind, w, eps, h = read
        _f32(in_w, "stream input weights", (S,))
        kind = _NORM_KINDS[norm_kind]
        _gpu(h, "normed rows")
        if tuple(h.shape) != (T, n) or (kind == 2 and h.dtype != torch.float32):
            raise InvalidArgument(f"normed rows {list(h.shape)} {h.dtype} do not fit {[T, n]}")
        if kind != 2:
            _f32(w, "norm weight", (n,))
        h_code = _code(h, "normed rows")
    if T == 0:
        return
    _call(_lib("hyper").tie_hyper_connection, "hyper_connection", streams.data_ptr(), streams.stride(0), S, int(from_x),
          _ptr(x), int(fold), _ptr(y), plane_stride, planes, _ptr(mix), _ptr(out_w), _ptr(in_w), _ptr(w), float(eps),
          kind, _ptr(h), h_code, T, n, _stream())


# ------------------------------------------------- short convolutions, the gated delta rule
CONV_MAX_TAPS = 8            # CONV_MAX_TAPS of csrc/delta_rule.hip
DELTA_RULE_MAX_DIM = 256     # key rows of a state the scan kernel keeps in registers (an eighth of them a lane)


def conv_qkv(u: torch.Tensor, weight: torch.Tensor, taps: int, state: Optional[torch.Tensor], batch, sizes,
             out: torch.Tensor, q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
             counts=None, eps: float = 0.0) -> None:
    """The short causal convolution of an attention's projected q, k and v, and the norms over a whole projection.

    ``u``: float32 rows ``[T, >= nq + nk + nv]``, ``sizes`` = ``(nq, nk, nv)``; ``weight`` float32 ``[C, taps]``
    (the last tap is the current token's); ``state`` ``[slots, taps - 1, C]`` holds every sequence's last inputs
    (read here; ``conv_state_update`` writes it). ``q_norm`` / ``k_norm`` (float32 ``[nq]`` / ``[nk]``): q and k are
    divided by their root mean square over all heads at once (over ``counts`` = (values of q, of k) where fewer than
    the columns count) and multiplied by these. ``out``: float32 ``[T, C]`` rows."""
    nq, nk, nv = (int(v) for v in sizes)
    C = nq + nk + nv
    _gpu_strided(u, "projected rows")
    T = u.shape[0]
    if u.dtype != torch.float32 or u.dim() != 2 or u.shape[1] < C or u.stride(1) != 1:
        raise InvalidArgument(f"projected rows {list(u.shape)} {u.dtype} do not hold {C} float32 columns")
    _f32(weight, "convolution weights", (C, taps))
    _gpu_strided(out, "convolved rows")
    if out.dtype != torch.float32 or tuple(out.shape) != (T, C) or out.stride(1) != 1:
        raise InvalidArgument(f"convolved rows {list(out.shape)} do not fit {[T, C]}")
    if not 1 <= taps <= CONV_MAX_TAPS or C > ROW_IN_LDS_MAX:
        raise InvalidArgument(f"a convolution of {taps} taps over {C} channels exceeds {CONV_MAX_TAPS} taps or "
                              f"{ROW_IN_LDS_MAX} channels")
    if taps > 1:
        _f32(state, "convolution state")
        if tuple(state.shape[1:]) != (taps - 1, C):
            raise InvalidArgument(f"convolution state {list(state.shape)} does not fit {[taps - 1, C]} a slot")
    if q_norm is not None:
        _f32(q_norm, "q norm weight", (nq,))
    if k_norm is not None:
        _f32(k_norm, "k norm weight", (nk,))
    count_q, count_k = counts if counts is not None else (nq, nk)
    if T == 0:
        return
    _call(_lib("delta_rule").tie_conv_qkv, "conv_qkv", u.data_ptr(), u.stride(0), weight.data_ptr(), taps, _ptr(state),
          batch.state_slots.data_ptr(), batch.seq_of_row.data_ptr(), batch.query_start.data_ptr(), T, nq, nk, nv,
          _ptr(q_norm), _ptr(k_norm), float(count_q), float(count_k), float(eps), out.data_ptr(), out.stride(0),
          _stream())


def conv_state_update(u: torch.Tensor, taps: int, state: torch.Tensor, batch, channels: int) -> None:
    """After a step: every sequence's slot of ``state`` ``[slots, taps - 1, C]`` holds its last ``taps - 1`` inputs
    (rows of ``u``, or what the state held where the step brought fewer)."""
    if taps <= 1:
        return
    _gpu_strided(u, "projected rows")
    _f32(state, "convolution state")
    if u.dtype != torch.float32 or u.shape[1] < channels or tuple(state.shape[1:]) != (taps - 1, channels):
        raise InvalidArgument(f"rows {list(u.shape)} / state {list(state.shape)} do not fit {channels} channels, {taps} taps")
    if batch.num_seqs == 0:
        return
    _call(_lib("delta_rule").tie_conv_state_update, "conv_state_update", u.data_ptr(), u.stride(0), taps,
          state.data_ptr(), batch.state_slots.data_ptr(), batch.query_start.data_ptr(), batch.num_seqs, channels,
          _stream())


def delta_prepare(u: torch.Tensor, weight: torch.Tensor, taps: int, state: Optional[torch.Tensor], batch,
                  a: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor, kv_heads: int, heads: int, key_dim: int,
                  value_dim: int, out: torch.Tensor) -> None:
    """What the gated delta rule takes of every token, from the projections' float32 sums.

    ``u`` rows ``[q (G d) | k (G d) | v (H e) | b (H)]``: q, k, v through the short convolution and silu, q and k
    made unit vectors per head (q also times ``d ** -0.5``), ``beta = sigmoid(b)``; ``a`` rows ``[H d]``: the decays
    ``exp(-exp(A_log[head]) * softplus(a + dt_bias))``. ``out`` rows: ``[q | k | v | decay | beta]`` float32."""
    G, H, d, e = kv_heads, heads, key_dim, value_dim
    C = 2 * G * d + H * e
    _gpu_strided(u, "projected rows")
    _gpu_strided(a, "decay rows")
    T = u.shape[0]
    if u.dtype != torch.float32 or u.shape[1] < C + H or a.dtype != torch.float32 or tuple(a.shape) != (T, H * d):
        raise InvalidArgument(f"projected rows {list(u.shape)} / decay rows {list(a.shape)} do not fit the heads")
    _f32(weight, "convolution weights", (C, taps))
    _f32(A_log, "A_log", (H,))
    _f32(dt_bias, "dt_bias", (H * d,))
    _f32(out, "delta rule rows", (T, C + H + H * d))
    if not 1 <= taps <= CONV_MAX_TAPS or C > ROW_IN_LDS_MAX:
        raise InvalidArgument(f"a convolution of {taps} taps over {C} channels exceeds what the kernel takes")
    if taps > 1:
        _f32(state, "convolution state")
        if tuple(state.shape[1:]) != (taps - 1, C):
            raise InvalidArgument(f"convolution state {list(state.shape)} does not fit {[taps - 1, C]} a slot")
    if T == 0:
        return
    _call(_lib("delta_rule").tie_delta_prepare, "delta_prepare", u.data_ptr(), u.stride(0), weight.data_ptr(), taps,
          _ptr(state), batch.state_slots.data_ptr(), batch.seq_of_row.data_ptr(), batch.query_start.data_ptr(),
          a.data_ptr(), a.stride(0), A_log.data_ptr(), dt_bias.data_ptr(), T, G, H, d, e, out.data_ptr(),
          out.stride(0), _stream())


DELTA_CHUNK_ROWS = 256                 # rows of a chunk of the gated delta rule's chunked walk
DELTA_CHUNKS_FROM = 1024               # a step's longest portion from which the rule runs in chunks (three launches)
DELTA_CHUNK_SCRATCH_MAX = 1 << 30      # bytes of chunk states above which a step walks its sequences whole


def gated_delta_scan(tok: torch.Tensor, out: torch.Tensor, state: torch.Tensor, batch, kv_heads: int, heads: int,
                     key_dim: int, value_dim: int, chunks: Optional[ScanChunks] = None, scratch=None) -> None:
    """The gated delta rule, token by token through each sequence's state ``[slots, H, d, e]`` (float32):
    ``S <- decay * S`` row by row; ``u = beta * (v - S^T k)``; ``S <- S + k u^T``; ``o = S^T q``. ``tok``: the rows of
    ``delta_prepare``; ``out`` float32 ``[T, H e]``.

    With ``chunks`` (``scan_chunks``; ``scratch(name, shape, dtype)`` hands out the memory for the chunks' states)
    the rows run chunk beside chunk in three launches. A token's step is linear in the state,
    ``S_t = (I - beta k k^T) diag(decay) S_(t-1) + beta k v^T``, so a chunk is ``S_end = P S_start + L``: every chunk
    walks from a zero state with ``d`` more columns that start as the identity and take no values (they end as
    ``P``), the chunks' states are combined in order, and every chunk walks again from its true start, with
    outputs. The same values up to rounding."""
    G, H, d, e = kv_heads, heads, key_dim, value_dim
    T = tok.shape[0]
    _f32(tok, "delta rule rows", (T, 2 * G * d + H * e + H + H * d))
    _f32(out, "delta rule output", (T, H * e))
    _f32(state, "delta rule state")
    if tuple(state.shape[1:]) != (H, d, e) or H % G or d > DELTA_RULE_MAX_DIM:
        raise InvalidArgument(f"a state {list(state.shape)} does not fit {H} heads of {d} x {e} (keys up to "
                              f"{DELTA_RULE_MAX_DIM}, {G} key heads)")
    if batch.num_seqs == 0:
        return
    if chunks is not None and chunks.count * H * d * (e + d) * 4 <= DELTA_CHUNK_SCRATCH_MAX:
        ends = scratch("delta_rule.chunk_ends", (chunks.count, H, d, e + d), torch.float32)
        starts = scratch("delta_rule.chunk_starts", (chunks.count, H, d, e), torch.float32)
        _call(_lib("delta_rule").tie_gated_delta_scan_chunked, "gated_delta_scan_chunked", tok.data_ptr(),
              tok.stride(0), out.data_ptr(), out.stride(0), state.data_ptr(), batch.state_slots.data_ptr(),
              batch.num_seqs, chunks.items.data_ptr(), chunks.first_item.data_ptr(), chunks.count, ends.data_ptr(),
              starts.data_ptr(), G, H, d, e, _stream())
        return
    _call(_lib("delta_rule").tie_gated_delta_scan, "gated_delta_scan", tok.data_ptr(), tok.stride(0), out.data_ptr(),
          out.stride(0), state.data_ptr(), batch.query_start.data_ptr(), batch.state_slots.data_ptr(), batch.num_seqs,
          G, H, d, e, _stream())


def grouped_gated_rms_norm(o: torch.Tensor, weight: torch.Tensor, eps: float, gate: torch.Tensor, out: torch.Tensor,
                           groups: int) -> None:
    """out = o / rms(o over each of ``groups`` equal groups of columns) * weight[column in its group] * sigmoid(gate).
    ``o`` float32 ``[T, n]``, ``gate`` float32 rows of n (a view whose rows may lie further apart)."""
    _f32(o, "gated norm input")
    T, n = o.shape
    if groups <= 0 or n % groups:
        raise InvalidArgument(f"{n} columns are not {groups} equal groups")
    _f32(weight, "gated norm weight", (n // groups,))
    _gpu_strided(gate, "gate rows")
    if gate.dtype != torch.float32 or tuple(gate.shape) != (T, n) or gate.stride(1) != 1:
        raise InvalidArgument(f"gate rows {list(gate.shape)} {gate.dtype} do not fit float32 {[T, n]}")
    _gpu(out, "gated norm output")
    if tuple(out.shape) != (T, n):
        raise InvalidArgument(f"gated norm output {list(out.shape)} does not match input {[T, n]}")
    if T == 0:
        return
    _call(_lib("delta_rule").tie_grouped_gated_rms_norm, "grouped_gated_rms_norm", o.data_ptr(), o.stride(0),
          weight.data_ptr(), float(eps), gate.data_ptr(), gate.stride(0), out.data_ptr(),
          _code(out, "gated norm output"), T, groups, n // groups, _stream())


# ------------------------------------------------- latent attention
def latent_prepare(proj: torch.Tensor, latent_weight: torch.Tensor, eps: float, angles: Optional[torch.Tensor],
                   rotary_dim: int, pairing: str, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], block_size: int, write_kv: bool, q_plain: torch.Tensor,
                   q_latent: torch.Tensor, heads: int, dim: int, rot_dim: int, kv_rank: int,
                   latent_rows: Optional[torch.Tensor] = None) -> None:
    """Cache rows and query parts of a latent attention from the projection's float32 rows
    ``[q: H x (dim + rot_dim) | latent (kv_rank) | rotated key part (rot_dim) | ...]``.

    The latent is RMS-normed with ``latent_weight``; the key cache (one head of size D >= kv_rank + rot_dim) gets
    ``[latent | rotated key part | zeros]``, the value cache ``[latent | zeros]``. ``q_plain`` ``[T, H dim]`` gets
    the unrotated query parts, ``q_latent`` ``[T, H D]`` the rotated ones at columns ``kv_rank ..`` of every head
    (zeros behind; columns below ``kv_rank`` are left for the product that takes the plain parts there).
    ``latent_rows`` (float32 ``[T, >= kv_rank + rot_dim]``, rows possibly further apart): the latent and the key part
    where they do not follow the queries in ``proj`` (queries that come from a product of their own)."""
    _gpu_strided(proj, "projected rows")
    T = proj.shape[0]
    H, d, r, kr = heads, dim, rot_dim, kv_rank
    D = q_latent.shape[1] // H
    if proj.dtype != torch.float32 or proj.shape[1] < H * (d + r) + (0 if latent_rows is not None else kr + r) or \
            proj.stride(1) != 1:
        raise InvalidArgument(f"projected rows {list(proj.shape)} {proj.dtype} do not hold the queries and the latent")
    if latent_rows is not None:
        _gpu_strided(latent_rows, "latent rows")
        if latent_rows.dtype != torch.float32 or latent_rows.dim() != 2 or latent_rows.shape[0] != T or \
                latent_rows.shape[1] < kr + r or latent_rows.stride(1) != 1:
            raise InvalidArgument(f"latent rows {list(latent_rows.shape)} {latent_rows.dtype} do not hold the latent "
                                  f"and the key part of {T} tokens")
    _gpu(q_plain, "plain query parts")
    _gpu(q_latent, "latent queries")
    if tuple(q_plain.shape) != (T, H * d) or tuple(q_latent.shape) != (T, H * D) or D < kr + r or \
            q_plain.dtype != q_latent.dtype:
        raise InvalidArgument(f"query buffers {list(q_plain.shape)} / {list(q_latent.shape)} do not fit the heads")
    _f32(latent_weight, "latent norm weight", (kr,))
    if pairing not in ("rotate_half", "interleaved"):
        raise InvalidArgument(f"pairs rotate as 'rotate_half' or 'interleaved', not '{pairing}'")
    if rotary_dim:
        _f32(angles, "rope angles", (T, rotary_dim))
    cache_code = _code(q_plain, "queries")
    if write_kv:
        _i32(slots, "slot mapping", T)
        _check_cache(k_cache, v_cache, 1, block_size, D)
        cache_code = _cache_code(k_cache, q_plain, "k cache")
    if T == 0:
        return
    _call(_lib("latent").tie_latent_prepare, "latent_prepare", proj.data_ptr(), proj.stride(0),
          latent_rows.data_ptr() if latent_rows is not None else None,
          latent_rows.stride(0) if latent_rows is not None else 0, latent_weight.data_ptr(),
          float(eps), _ptr(angles) if rotary_dim else None, int(rotary_dim), int(pairing == "interleaved"),
          _ptr(slots) if write_kv else None, _ptr(k_cache) if write_kv else None, _ptr(v_cache) if write_kv else None,
          cache_code, block_size, int(write_kv), q_plain.data_ptr(), q_latent.data_ptr(), _code(q_plain, "queries"),
          T, H, d, r, kr, D, _stream())


def rms_norm_columns(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """``out = RMSNorm(x) * weight`` over float32 rows ``x [T, n]`` that may lie further apart than ``n`` (the first
    columns of wider rows); ``out`` ``[T, n]`` dense."""
    _gpu_strided(x, "rows to norm")
    _gpu(out, "normed rows")
    if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1 or tuple(out.shape) != tuple(x.shape):
        raise InvalidArgument(f"rms_norm_columns: rows {list(x.shape)} {x.dtype}, out {list(out.shape)}")
    T, n = x.shape
    _f32(weight, "norm weight", (n,))
    if T == 0:
        return
    _call(_lib("latent").tie_rms_norm_columns, "rms_norm_columns", x.data_ptr(), x.stride(0), weight.data_ptr(),
          float(eps), out.data_ptr(), _code(out, "normed rows"), T, n, _stream())


def head_linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> None:
    """``out[t, h] = w[h] @ x[t, h]`` for every head: ``x`` ``[T, H, K]``, ``w`` ``[H, N, K]``, ``out`` ``[T, H, N]``
    (views whose rows and heads may lie further apart; the last dimension is dense), float32 sums; with ``gate``
    (float32 ``[T, H, N]`` view) the result is multiplied by ``sigmoid(gate)``."""
    for t, name in ((x, "head inputs"), (out, "head outputs")):
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise KernelUnavailable(f"{name} must be a tensor on a GPU: the engine's kernels have no CPU fallback")
        if t.dim() != 3 or t.stride(2) != 1:
            raise InvalidArgument(f"{name} {list(t.shape)} must be [rows, heads, width] with a dense last dimension")
    _gpu(w, "head matrices")
    T, H, K = x.shape
    N = w.shape[1]
    if tuple(w.shape) != (H, N, K) or tuple(out.shape) != (T, H, N):
        raise InvalidArgument(f"head matrices {list(w.shape)} do not take {list(x.shape)} to {list(out.shape)}")
    if gate is not None:
        if not gate.is_cuda or gate.dim() != 3:
            raise InvalidArgument("head gates must be a [rows, heads, width] tensor on the GPU")
        if gate.dtype != torch.float32 or tuple(gate.shape) != (T, H, N) or gate.stride(2) != 1:
            raise InvalidArgument(f"head gates {list(gate.shape)} {gate.dtype} do not fit float32 {[T, H, N]}")
    if T == 0:
        return
    _call(_lib("latent").tie_head_linear, "head_linear", x.data_ptr(), _code(x, "head inputs"), x.stride(0), x.stride(1),
          w.data_ptr(), _code(w, "head matrices"), out.data_ptr(), _code(out, "head outputs"), out.stride(0),
          out.stride(1), _ptr(gate), gate.stride(0) if gate is not None else 0,
          gate.stride(1) if gate is not None else 0, T, H, N, K, _stream())
