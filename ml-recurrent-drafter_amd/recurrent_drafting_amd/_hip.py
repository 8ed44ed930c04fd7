"""ctypes binding of libredrafter_hip.so (the C ABI declared in include/redrafter_hip.h).

PyTorch is used only for device memory and streams: tensors are handed over as raw device pointers
plus sizes/strides, and every launch goes to torch's current HIP stream.  There is no fallback: if
the library is missing, or a tensor is not on the GPU, the call raises.
"""

from __future__ import annotations

import ctypes as C
import os

import torch

import sys

# The library built from csrc/ sits beside this file.  RD_HIP_LIBRARY names another build of it (an
# A/B of two builds on one machine); whoever loads one is told so on stderr, and the test suite
# refuses to run on it (tests/conftest.py).
_DEFAULT_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libredrafter_hip.so")
_LIB_PATH = os.environ.get("RD_HIP_LIBRARY") or _DEFAULT_LIB_PATH
_lib = None
ABI_VERSION = 106  # RD_ABI_VERSION of include/redrafter_hip.h that _PROTOTYPES below was written against

RD_BF16, RD_F16, RD_F32 = 0, 1, 2
_DTYPES = {torch.bfloat16: RD_BF16, torch.float16: RD_F16, torch.float32: RD_F32}

_P, _I, _L, _Z, _F = C.c_void_p, C.c_int, C.c_int64, C.c_size_t, C.c_float

_PROTOTYPES = {
    "rd_version": (C.c_int, []),
    "rd_last_error": (C.c_char_p, []),
    "rd_timing_enable": (_I, [_I]),
    "rd_timing_select": (_I, [C.c_char_p]),
    "rd_timing_sample": (_I, [_I]),
    "rd_timing_null_kernel_us": (_I, [_I, _P, C.POINTER(C.c_float)]),
    "rd_timing_collect": (_I, [C.c_char_p, _Z]),
    "rd_tree_workspace_bytes": (_Z, [_I, _I, _I]),
    "rd_tree_build": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _Z, _P]),
    "rd_tree_mask": (_I, [_P, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _P, _P]),
    "rd_unpack_rows": (_I, [_P, _L, _L, _P, _L, _I, _I, _I, _P, _L, _L, _P, _P]),
    "rd_argmax_rows": (_I, [_P, _I, _L, _L, _L, _P, _P, _P]),
    "rd_accept_greedy": (_I, [_P, _P, _L, _P, _I, _I, _I, _P, _P, _P, _P, _P]),
    "rd_count_left_paddings": (_I, [_P, _L, _L, _I, _L, _P, _P]),
    "rd_position_ids": (_I, [_P, _L, _L, _I, _L, _P, _L, _I, _P, _P]),
    "rd_realign_plan_ints": (_Z, [_I, _I]),
    "rd_realign_plan": (_I, [_P, _L, _L, _P, _P, _P, _P, _I, _I, _I, _L, _P, _P, _P, _P, _P, _P]),
    "rd_kv_unpack": (_I, [_P, _I, _I, _I, _L, _L, _L, _P, _I, _I, _P]),
    "rd_kv_compact": (_I, [_P, _I, _I, _I, _L, _L, _L, _I, _P, _P]),
    "rd_kv_append": (_I, [_P, _I, _I, _I, _L, _L, _I, _P, _P]),
    "rd_kv_materialize_plan_ints": (_Z, [_I]),
    "rd_kv_materialize": (_I, [_P, _I, _I, _I, _L, _L, _L, _P, _P, _P]),
    "rd_add_rms_norm": (_I, [_P, _L, _P, _L, _P, _P, _L, _P, _L, _I, _L, _I, _F, _P]),
    "rd_silu_mul": (_I, [_P, _P, _L, _P, _L, _I, _L, _I, _P]),
    "rd_silu_add": (_I, [_P, _L, _P, _L, _P, _L, _P, _L, _I, _I, _L, _I, _P]),
    "rd_rope_append": (
        _I,
        [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P, _L, _P, _L, _P, _P, _P, _P, _P, _L, _L, _P, _P, _P],
    ),
    "rd_attn_plan_ints": (_Z, [_I, _I, _I]),
    "rd_attn_bits_words": (_Z, [_I, _I, _I]),
    "rd_attn_prepare": (_I, [_P, _L, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P]),
    "rd_tree_attn_prepare": (_I, [_P, _P, _P, _P, _I, _L, _L, _L, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "rd_attention_workspace_bytes": (_Z, [_I, _I, _I, _I, _I]),
    "rd_verify_attention": (
        _I,
        [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P, _P, _P, _Z, _I, _P, _P],
    ),
    "rd_rope_verify_attention_eligible": (_I, [_I, _I, _I, _I]),
    "rd_rope_verify_attention": (
        _I,
        [_P, _P, _P, _P, _P, _P, _P, _P, _L, _P, _L, _P, _P, _P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F,
         _P, _P, _P, _Z, _P, _P],
    ),
    "rd_causal_mask": (_I, [_P, _I, _L, _I, _L, _L, _P, _P]),
    "rd_verify_row_stats": (_I, [_P, _I, _L, _L, _I, _I, _F, _F, _P, _I, _P]),
    "rd_accept_sample": (
        _I,
        [_P, _P, _P, _P, _I, _P, _P, _I, _P, _F, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P],
    ),
    "rd_residual_probs": (
        _I,
        [_P, _P, _P, _I, _P, _P, _I, _P, _F, _P, _P, _P, _P, _I, _I, _I, _I, _P, _P],
    ),
    "rd_beam_topk_workspace_bytes": (_Z, [_I, _I]),
    "rd_beam_topk": (
        _I,
        [_P, _I, _L, _L, _I, _I, _I, _P, _I, _F, _P, _I, _P, _P, _P, _P, _P, _L, _P, _Z, _I, _P],
    ),
    "rd_beam_init": (_I, [_P, _L, _P, _I, _I, _L, _F, _P, _P, _P, _L, _P, _I, _P]),
    "rd_beam_topk_static": (
        _I,
        [_P, _I, _L, _L, _I, _I, _I, _P, _I, _F, _P, _I, _P, _P, _P, _P, _P, _L, _I, _P],
    ),
}


def library_path() -> str:
    return _LIB_PATH


def is_default_library() -> bool:
    """False when RD_HIP_LIBRARY points the package at another build of the library."""
    return os.path.realpath(_LIB_PATH) == os.path.realpath(_DEFAULT_LIB_PATH)


def lib():
    """Loads the shared library on first use."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with "
                "`python ml-recurrent-drafter_amd/build_hip.py` (needs hipcc); "
                "there is no CPU or PyTorch fallback for the HIP kernels"
            )
        handle = C.CDLL(_LIB_PATH)
        if not is_default_library():
            print(f"recurrent_drafting_amd: RD_HIP_LIBRARY is set, using {_LIB_PATH} instead of the in-tree "
                  "library", file=sys.stderr, flush=True)
        handle.rd_version.restype = C.c_int
        found = handle.rd_version()
        if found != ABI_VERSION:
            raise RuntimeError(
                f"{_LIB_PATH} has interface version {found}, this package was written against {ABI_VERSION}: "
                "rebuild it with `python ml-recurrent-drafter_amd/build_hip.py`")
        for name, (res, args) in _PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().rd_last_error().decode()
        raise RuntimeError(f"libredrafter_hip error {rc}: {msg}")


def ptr(t: torch.Tensor | None):
    """Device pointer of a tensor (None -> NULL).  Refuses host tensors: the kernels would fault."""
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError(
            "the HIP hot path needs tensors on the GPU (got a CPU tensor); "
            "there is no CPU fallback in this package"
        )
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def stream():
    """Handle of torch's current stream on the current device.  Every launch asks for it, so the two
    direct calls are used where this torch build has them (a few tenths of a microsecond against
    about three for `torch.cuda.current_stream()`)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; expected bfloat16, float16 or float32") from None


def timing_sample(every: int) -> None:
    """Time every `every`-th qualifying launch only (1: all of them)."""
    check(lib().rd_timing_sample(int(every)))


def timing_enable(on: bool) -> None:
    """Per-kernel HIP-event timing inside the library (a measurement aid; off by default)."""
    check(lib().rd_timing_enable(int(on)))


def timing_select(kernel: str | None) -> None:
    """Time only the named kernel (None: all kernels)."""
    check(lib().rd_timing_select(kernel.encode() if kernel else None))


def timing_null_kernel_us(launches: int = 64) -> float:
    """Event-to-event time of an empty kernel: the fixed overhead inside every timed figure."""
    out = C.c_float(0.0)
    check(lib().rd_timing_null_kernel_us(launches, stream(), C.byref(out)))
    return float(out.value)


def timing_collect() -> dict:
    """{kernel name: (launches, total milliseconds)} since the last call; waits for the events."""
    buf = C.create_string_buffer(1 << 16)
    check(lib().rd_timing_collect(buf, len(buf)))
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, total = line.split()
        out[name] = (int(count), float(total))
    return out


def aligned_rows(x: torch.Tensor) -> torch.Tensor:
    """(rows, V) view whose rows start on 16-byte boundaries (the row kernels load 16-byte vectors).
    Already-aligned tensors pass through; others are copied into a padded buffer once."""
    es = x.element_size()
    if x.stride(1) == 1 and (x.stride(0) * es) % 16 == 0 and x.data_ptr() % 16 == 0:
        return x
    rows, v = x.shape
    per = 16 // es
    padded = torch.empty((rows, (v + per - 1) // per * per), dtype=x.dtype, device=x.device)
    padded[:, :v] = x
    return padded[:, :v]
