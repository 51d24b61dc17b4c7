"""Decode attention on MI355X: one new query token per sequence against the key/value cache
(the adapter's decode branch, moba/wrapper.py:76-82, which calls flash_attn_func in the
reference).  The HIP kernel reads K and V of the cache once, in place, with grouped-query heads."""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib

SUPPORTED_GROUP_SIZES = (1, 2, 4, 8)


def supported(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> bool:
    """True when decode_attention can take these tensors ([B,H,1,D] and [B,Hkv,Skv,D])."""
    if not (query.is_cuda and key.is_cuda and value.is_cuda):
        return False
    if query.dtype not in (torch.bfloat16, torch.float16) or key.dtype != query.dtype or value.dtype != query.dtype:
        return False
    if query.dim() != 4 or key.dim() != 4 or key.shape != value.shape:
        return False
    b, h, q_len, d = query.shape
    if q_len != 1 or d != 128 or key.shape[0] != b or key.shape[3] != d or key.shape[2] == 0:
        return False
    return key.shape[1] > 0 and h % key.shape[1] == 0 and h // key.shape[1] in SUPPORTED_GROUP_SIZES


def _rows_in_place(t: torch.Tensor) -> torch.Tensor:
    """A [B,Hkv,Skv,D] tensor whose key rows are contiguous and D apart, with 16-byte friendly strides."""
    d = t.shape[3]
    ok = t.stride(3) == 1 and t.stride(2) == d and t.stride(0) % 8 == 0 and t.stride(1) % 8 == 0 and t.data_ptr() % 16 == 0
    return t if ok else t.contiguous()


def decode_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                     scaling: Optional[float] = None) -> torch.Tensor:
    """query [B,H,1,D], key/value [B,Hkv,Skv,D] -> [B,1,H,D] (the layout the adapter returns).
    Softmax scale ``scaling`` (default D**-0.5); every cached key is visible."""
    if not supported(query, key, value):
        raise ValueError("decode_attention needs bf16/fp16 GPU tensors, one query token, head_dim 128 and "
                         "1, 2, 4 or 8 query heads per key/value head")
    lib = _lib.load()
    b, h, _, d = query.shape
    hkv, skv = key.shape[1], key.shape[2]
    q = query if (query.stride(3) == 1 and query.stride(0) % 8 == 0 and query.stride(1) % 8 == 0
                  and query.data_ptr() % 16 == 0) else query.contiguous()
    k, v = _rows_in_place(key), _rows_in_place(value)
    if k.stride() != v.stride():
        k, v = k.contiguous(), v.contiguous()
    splits = lib.moba_decode_splits(b, hkv, skv)
    dev = query.device
    part_o = torch.empty((b * h * splits, d), dtype=torch.float32, device=dev)
    part_lse = torch.empty((b * h * splits,), dtype=torch.float32, device=dev)
    out = torch.empty((b, 1, h, d), dtype=query.dtype, device=dev)
    scale = float(scaling) if scaling is not None else d ** -0.5
    dtype = _lib.DTYPE_F16 if query.dtype == torch.float16 else _lib.DTYPE_BF16
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    _lib.check(lib.moba_decode(p(q), p(k), p(v), p(out), p(part_o), p(part_lse), b, h, hkv, skv, d,
                               q.stride(0), q.stride(1), k.stride(0), k.stride(1), scale, dtype, stream),
               "moba_decode")
    return out
