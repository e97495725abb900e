"""ctypes binding of ``libdaisy_hip.so`` (declared in ``include/daisy_hip.h``).

The library is loaded from ``daisy_amd/csrc`` where ``python -m daisy_amd.build``
puts it.  There is no fallback: if the library is missing, or a tensor is not on
a GPU, the call raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libdaisy_hip.so")
_lib: Optional[ctypes.CDLL] = None

ABI_VERSION = 5
LINEAR_MAX_ROWS = 8
STATUS_POSITION_PAST_TABLES = 1
DECODE_STATIC_SCRATCH_BYTES = 4 << 20

_I64P = POINTER(c_int64)

# name -> (restype, argtypes); mirrors include/daisy_hip.h one to one.
SIGNATURES = {
    "daisy_last_error": (c_char_p, []),
    "daisy_abi_version": (c_int, []),
    "daisy_prefill_fwd": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k, v (+strides)
        c_void_p, c_void_p, c_void_p,                           # cos, sin, doc_start
        c_void_p, _I64P, c_void_p, _I64P,                       # o, k_out (+strides)
        c_int, c_int, c_int, c_int,                             # B, T, H, D
        c_int, c_float, c_int, c_void_p]),                      # window, scale, flags, stream
    "daisy_prefill_fwd_f32": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k, v (+strides), fp32
        c_void_p, c_void_p, c_void_p,                           # cos, sin, doc_start
        c_void_p, _I64P, c_void_p, _I64P,                       # o, k_out (+strides), fp32
        c_int, c_int, c_int, c_int,                             # B, T, H, D
        c_int, c_float, c_void_p]),                             # window, scale, stream
    "daisy_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "daisy_decode_fwd": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k_new, v_new (+strides)
        c_void_p, _I64P, c_void_p, _I64P,                       # k_cache, v_cache (+strides)
        c_void_p, c_void_p,                                     # cos_row, sin_row
        c_void_p, _I64P,                                        # o (+strides)
        c_int, c_int, c_int,                                    # B, H, D
        c_int, c_int, c_int,                                    # n_rows, new_idx, write_back
        c_float, c_int,                                         # scale, nsplit
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_decode_fwd_f32": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k_new, v_new (+strides), fp32
        c_void_p, _I64P, c_void_p, _I64P,                       # k_cache, v_cache (+strides), fp32
        c_void_p, c_void_p,                                     # cos_row, sin_row
        c_void_p, _I64P,                                        # o (+strides)
        c_int, c_int, c_int,                                    # B, H, D
        c_int, c_int, c_int,                                    # n_rows, new_idx, write_back
        c_float, c_void_p]),                                    # scale, stream
    "daisy_decode_noalloc_init": (c_int, []),
    "daisy_decode_fwd_noalloc": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k_new, v_new (+strides)
        c_void_p, _I64P, c_void_p, _I64P,                       # k_cache, v_cache (+strides)
        c_void_p, c_void_p,                                     # cos_row, sin_row
        c_void_p, _I64P,                                        # o (+strides)
        c_int, c_int, c_int,                                    # B, H, D
        c_int, c_int, c_int,                                    # n_rows, new_idx, write_back
        c_float, c_int, c_void_p]),                             # scale, nsplit, stream
    "daisy_decode_fwd_at": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k_new, v_new (+strides)
        c_void_p, _I64P, c_void_p, _I64P,                       # k_cache, v_cache (+strides)
        c_void_p, _I64P,                                        # o (+strides)
        c_int, c_int, c_int,                                    # B, H, D
        c_int, c_void_p,                                        # ring_rows, pos (device int32)
        c_float, c_int,                                         # scale, nsplit
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_attn_step_fwd": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,      # q, k, v rows of the projection (+strides)
        c_void_p, _I64P, c_void_p,                              # ve, ve strides, gate
        c_void_p, c_void_p, c_int,                              # cos, sin, table_rows
        c_int, c_void_p, c_void_p, c_float,                     # pos, pos_dev, status, eps
        c_void_p, _I64P, c_void_p, _I64P, c_int,                # k_cache, v_cache (+strides), cache_is_f16
        c_void_p, _I64P,                                        # o (+strides)
        c_int, c_int, c_int, c_int,                             # B, H, D, ring_rows
        c_float, c_int,                                         # scale, nsplit
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_kda_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "daisy_kda_chunk_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p,                           # q, k, v
        c_void_p, c_int, c_void_p,                              # g, g_is_bf16, beta
        c_void_p, c_void_p, c_void_p,                           # initial_state, o, final_state
        c_int, c_int, c_int, c_int, c_int, c_int,               # B, T, H, Dk, Dv, chunk
        c_float, c_int, c_float,                                # scale, l2norm_qk, l2_eps
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_kda_varlen_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "daisy_kda_chunk_varlen_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p,                           # q, k, v
        c_void_p, c_int, c_void_p,                              # g, g_is_bf16, beta
        c_void_p, c_int,                                        # cu_seqlens (device int32), n_seq
        c_void_p, c_void_p, c_void_p,                           # initial_state, o, final_state
        c_int, c_int, c_int, c_int, c_int,                      # T, H, Dk, Dv, chunk
        c_float, c_int, c_float,                                # scale, l2norm_qk, l2_eps
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_kda_recurrent_varlen_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,  # q, k, v, g, g_is_bf16, beta
        c_void_p, c_int,                                        # cu_seqlens (device int32), n_seq
        c_void_p, c_void_p, c_void_p,                           # initial_state, o, final_state
        c_int, c_int, c_int, c_int,                             # T, H, Dk, Dv
        c_float, c_int, c_float, c_void_p]),                    # scale, l2norm_qk, l2_eps, stream
    "daisy_kda_recurrent_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,  # q, k, v, g, g_is_bf16, beta
        c_void_p, c_void_p, c_void_p,                           # initial_state, o, final_state
        c_int, c_int, c_int, c_int, c_int,                      # B, T, H, Dk, Dv
        c_float, c_int, c_float, c_void_p]),                    # scale, l2norm_qk, l2_eps, stream
    "daisy_kda_gate_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p,                 # g, A_log, bias, out
        c_int64, c_int, c_int, c_int,                           # rows, H, Dk, io_is_bf16
        c_float, c_float, c_void_p]),                           # softplus beta, threshold, stream
    "daisy_short_conv_fwd": (c_int, [
        c_void_p, _I64P, c_void_p, c_void_p, c_void_p,          # x (+ strides), weight, bias, cache_in
        c_void_p, _I64P, c_void_p,                              # y (+ strides), cache_out
        c_int, c_int, c_int, c_int, c_int, c_void_p]),          # B, T, C, K, apply_silu, stream
    "daisy_gated_rmsnorm_fwd": (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_void_p]),
    "daisy_short_conv_varlen_fwd": (c_int, [
        c_void_p, c_int64, c_void_p, c_void_p,                  # x, x row stride, weight, bias
        c_void_p, c_int, c_void_p,                              # cu_seqlens (device int32), n_seq, cache_in
        c_void_p, c_int64, c_void_p,                            # y, y row stride, cache_out
        c_int, c_int, c_int, c_int, c_void_p]),                 # T, C, K, apply_silu, stream
    "daisy_linear_rows_fwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,   # x, w, y (+ row strides)
                                       c_int, c_int, c_int, c_void_p]),                          # M, N, K, stream
    "daisy_attn_layer_step_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "daisy_attn_layer_step_fwd": (c_int, [
        c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,   # x, w_qkv, w_out (+ row strides)
        c_void_p, _I64P, c_void_p,                               # ve, ve strides, gate
        c_void_p, c_void_p, c_int,                              # cos, sin, table_rows
        c_int, c_void_p, c_void_p, c_float,                     # pos, pos_dev, status, eps
        c_void_p, _I64P, c_void_p, _I64P, c_int,                # k_ring, v_ring (+strides), ring is fp16
        c_void_p, c_int64,                                      # y (+ row stride)
        c_int, c_int, c_int, c_int, c_int,                      # B, H, D, dim, ring_rows
        c_float, c_int,                                         # scale, nsplit
        c_void_p, c_size_t, c_void_p]),                         # workspace, bytes, stream
    "daisy_qkv_prep_fwd": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,         # q, k, v (+ strides)
        c_void_p, _I64P, c_void_p,                               # ve, ve strides, gate
        c_void_p, c_void_p, c_int,                              # cos, sin, pos0
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,         # q_out, k_out, v_out (+ strides)
        c_int, c_int, c_int, c_int, c_float, c_void_p]),        # B, T, H, D, eps, stream
    "daisy_qkv_prep_fwd_at": (c_int, [
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,         # q, k, v (+ strides)
        c_void_p, _I64P, c_void_p,                               # ve, ve strides, gate
        c_void_p, c_void_p, c_void_p, c_int, c_void_p,          # cos, sin, pos0 (device int32), table_rows, status
        c_void_p, _I64P, c_void_p, _I64P, c_void_p, _I64P,         # q_out, k_out, v_out (+ strides)
        c_int, c_int, c_int, c_int, c_float, c_void_p]),        # B, T, H, D, eps, stream
}


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Loads the shared library (once) and sets the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m daisy_amd.build` "
            "(there is no CPU or PyTorch fallback for the attention kernels)")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.daisy_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libdaisy_hip.so has ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().daisy_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


_STRIDE_ARRAYS: dict = {}


def strides(t: torch.Tensor, dims) -> ctypes.Array:
    """Element strides of the given dims as an int64 C array (read-only for the callee, so equal
    stride tuples share one array: decode loops ask for the same few over and over)."""
    st = t.stride()
    key = tuple(st[d] for d in dims)
    arr = _STRIDE_ARRAYS.get(key)
    if arr is None:
        if len(_STRIDE_ARRAYS) > 4096:
            _STRIDE_ARRAYS.clear()
        arr = _STRIDE_ARRAYS[key] = (c_int64 * len(key))(*key)
    return arr


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def require_gpu(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All tensors must live on one GPU; returns that device."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "daisy_amd kernels run on an AMD GPU only (got a tensor on "
                f"'{t.device}'); there is no CPU path")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise RuntimeError("no tensor given")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(dev: torch.device) -> int:
    """The ``hipStream_t`` of torch's current stream on ``dev`` as an integer."""
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def on_device(dev: torch.device):
    """Context that makes ``dev`` the current device for the launch; free when it already is."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _NO_GUARD
    return torch.cuda.device(dev)
