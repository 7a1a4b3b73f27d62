"""ctypes binding of libtgg_amd.so (the C ABI declared in include/tgg_amd.h).

There is no fallback: if the shared library is missing or a call fails, the
caller gets an exception.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_int, c_int64, c_void_p
from pathlib import Path
from typing import Optional

import torch

LIB_PATH = Path(__file__).resolve().parent / "libtgg_amd.so"

BF16, F16, E4M3, E5M2 = 0, 1, 2, 3
MAX_GROUPS = 1024  # TGG_MAX_GROUPS: plain 16-bit M-grouped and K-grouped GEMM
MAX_GROUPS_OTHER = 512  # TGG_MAX_GROUPS_OTHER: every other GEMM entry point
QUEUE_WORDS = 16  # TGG_QUEUE_WORDS: int32 words of the K-grouped kernels' work queue (zero before a launch, zero after)

_P, _I, _L = c_void_p, c_int, c_int64

# name -> argument types; every function returns int unless noted
SIGNATURES = {
    "tgg_m_grouped_gemm": [_P, _P, _P, _P, _I, _I, _L, _I, _I, _I, _I, _I, _P],
    "tgg_m_grouped_gemm_padded": [_P, _P, _P, _P, _I, _I, _L, _I, _I, _I, _I, _I, _P],
    "tgg_m_grouped_gemm_placed": [_P, _P, _P, _P, _I, _P, _I, _L, _I, _I, _I, _I, _P],
    "tgg_m_grouped_gemm_masked": [_P, _P, _P, _P, _I, _I, _L, _L, _I, _I, _I, _I, _I, _P],
    "tgg_k_grouped_gemm": [_P, _P, _P, _P, _P, _I, _I, _I, _L, _I, _I, _P],
    "tgg_k_grouped_gemm_queued": [_P, _P, _P, _P, _P, _I, _I, _I, _L, _I, _I, _P, _P],
    "tgg_m_grouped_gemm_fp8_channel": [_P, _P, _P, _P, _P, _P, _I, _I, _L, _I, _I, _I, _I, _I, _I, _P],
    "tgg_k_grouped_gemm_fp8_channel": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _L, _I, _I, _I, _P],
    "tgg_k_grouped_gemm_fp8_channel_queued": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _L, _I, _I, _I, _P, _P],
    "tgg_m_grouped_gemm_fp8_block": [_P, _P, _P, _P, _P, _P, _I, _I, _L, _I, _I, _I, _I, _I, _P],
    "tgg_m_grouped_gemm_fp8_block_placed": [_P, _P, _P, _P, _P, _P, _I, _P, _I, _L, _I, _I, _I, _I, _P],
    "tgg_trans_per_block_quant_expand_128x": [_P, _P, _P, _P, _I, _I, _L, _I, _L, _I, _P],
    "tgg_per_token_cast_to_fp8": [_P, _P, _P, _L, _I, _I, _I, _P],
    "tgg_per_block_cast_to_fp8": [_P, _P, _P, _I, _I, _I, _I, _P],
    "tgg_cvt_f32_to_fp8": [_P, _P, _L, _I, _P],
    "tgg_m_grouped_gemm_fp8_out": [_P, _P, _P, _P, _P, _I, _I, _L, _I, _I, _I, _I, _I, _I, _I, _P],
    "tgg_moe_sort_workspace_bytes": [_L, _I, _I, _P],
    "tgg_moe_permute_map": [_P, _L, _I, _I, _L, _P, _P, _I, _P, _L, _P],
    "tgg_moe_permute_map_static": [_P, _L, _I, _I, _L, _P, _P, _I, _P],
    "tgg_moe_permute_rows": [_P, _P, _P, _L, _I, _I, _I, _P],
    "tgg_moe_unpermute": [_P, _P, _P, _P, _L, _I, _I, _I, _P],
    "tgg_moe_unpermute_bwd": [_P, _P, _P, _P, _P, _P, _L, _I, _I, _I, _P],
    "tgg_debug_tile_order": [_P, _I, _I, _L, _L, _I, _I, _I, _I, _P, _L, _P],
    "tgg_debug_row_tiles": [_P, _I, _I, _L, _L, _I, _I, _P, _L, _P],
    "tgg_debug_queue_order": [_I, _I, _P],
    "tgg_debug_generic_extents": [_I, _P, _P, _I, _L, _L, _I, _I, _P],
    "tgg_set_option": [c_char_p, _I],
    "tgg_version": [],
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m triton_grouped_gemm_amd.build` "
                "(there is no non-HIP fallback)")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = c_int
        lib.tgg_last_error.argtypes = []
        lib.tgg_last_error.restype = c_char_p
        _lib = lib
    return _lib


def last_error() -> str:
    return load().tgg_last_error().decode()


def call(name: str, *args) -> None:
    rc = getattr(load(), name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed (code {rc}): {last_error()}")


def set_option(key: str, value: int) -> None:
    call("tgg_set_option", key.encode(), int(value))


def stream_of(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


_work_queues = {}


def work_queue(device: torch.device, queue: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The K-grouped kernels' tile counters for a launch on ``device``'s current stream: the caller's ``queue``
    (QUEUE_WORDS int32 on that device, zero, and not in use by a launch on another stream) or one the library keeps
    per (device, stream).  The kernels leave the words zero again, so the kept tensor is cleared once, when it is
    made, and a call costs no fill kernel and no allocation.  While the stream is being captured a tensor made here
    would belong to the graph's memory pool: the capture gets a fresh one (its fill is part of the graph) unless
    the caller brings its own."""
    if queue is not None:
        assert queue.is_cuda and queue.device == device and queue.dtype == torch.int32 and queue.is_contiguous() \
            and queue.numel() >= QUEUE_WORDS, f"queue must be {QUEUE_WORDS} contiguous int32 on {device}"
        return queue
    if torch.cuda.is_current_stream_capturing():
        return torch.zeros(QUEUE_WORDS, dtype=torch.int32, device=device)
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    q = _work_queues.get(key)
    if q is None:
        q = _work_queues[key] = torch.zeros(QUEUE_WORDS, dtype=torch.int32, device=device)
    return q


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise AssertionError("all tensors must live on the GPU (HIP device); this library has no CPU path")


DTYPE_CODE = {torch.bfloat16: BF16, torch.float16: F16}
FP8_CODE = {torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2}
