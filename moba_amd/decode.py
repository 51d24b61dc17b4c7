"""Decode attention on MI355X: new query tokens against the key/value cache (the adapter's decode
branch, moba/wrapper.py:76-82, which calls flash_attn_func in the reference: every cached key is
visible to a new token up to its own position).  One token: the HIP decode kernel reads K and V of
the cache once, in place, with grouped-query heads.  A few tokens: that kernel once per token.  Many
tokens (chunked prefill against a cache): the forward attention kernel's causal tiles on the tail of
the sequence."""

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


SHORT_QUERY = 16   # up to this many new tokens: one launch of the decode kernel per token


def chunk_supported(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> bool:
    """True when chunk_decode_attention can take these tensors ([B,H,q_len,D] and [B,Hkv,Skv,D], q_len <= Skv)."""
    if not (query.is_cuda and key.is_cuda and value.is_cuda):
        return False
    if query.dtype not in (torch.bfloat16, torch.float16) or key.dtype != query.dtype or value.dtype != query.dtype:
        return False
    if query.dim() != 4 or key.dim() != 4 or key.shape != value.shape:
        return False
    b, h, q_len, d = query.shape
    if d != 128 or key.shape[0] != b or key.shape[3] != d or not 0 < q_len <= key.shape[2]:
        return False
    return key.shape[1] > 0 and h % key.shape[1] == 0


_TAIL_TABLES = {}  # (kv_len, row tiles skipped, device) -> int32 tables of the causal tiles of a sequence's tail


def _tail_tables(kv_len: int, skip: int, tile_rows: int, device):
    """achunk_tok [2], self_tile_prefix [2], self_tile_chunk [m], chunk_direct [1] for one sequence of kv_len keys
    whose first `skip` row tiles do not exist; one small upload per distinct (length, skip)."""
    key = (kv_len, skip, str(device))
    hit = _TAIL_TABLES.get(key)
    if hit is None:
        if len(_TAIL_TABLES) >= 64:
            _TAIL_TABLES.pop(next(iter(_TAIL_TABLES)))
        m = -(-kv_len // tile_rows) - skip
        t = torch.tensor([0, kv_len, 0, m] + [0] * m + [1], dtype=torch.int32).to(device)
        hit = _TAIL_TABLES[key] = (t, m)
    return hit


def chunk_decode_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                           scaling: Optional[float] = None) -> torch.Tensor:
    """query [B,H,q_len,D]: the last q_len tokens of sequences whose keys and values [B,Hkv,Skv,D] the cache
    holds; token j attends the keys up to its own position Skv - q_len + j.  Returns [B,q_len,H,D]."""
    if not chunk_supported(query, key, value):
        raise ValueError("chunk_decode_attention needs bf16/fp16 GPU tensors, head_dim 128, no more query tokens than "
                         "keys and a whole number of query heads per key/value head")
    b, h, q_len, d = query.shape
    hkv, kv_len = key.shape[1], key.shape[2]
    if q_len <= SHORT_QUERY and h // hkv in SUPPORTED_GROUP_SIZES:
        first = kv_len - q_len + 1
        return torch.cat([decode_attention(query[:, :, j:j + 1], key[:, :, :first + j], value[:, :, :first + j], scaling)
                          for j in range(q_len)], dim=1)
    from . import moba_efficient as E
    lib = _lib.load()
    dev = query.device
    tile_rows = lib.moba_fwd_tile_rows()
    shift = kv_len - q_len
    skip = shift // tile_rows
    q_shift = skip * tile_rows
    pad = shift - q_shift                 # rows of the first tile that lie before the first query token
    tables, m = _tail_tables(kv_len, skip, tile_rows, dev)
    tp = tables.data_ptr()
    at = lambda i: ctypes.c_void_p(tp + 4 * i)
    scale = float(scaling) if scaling is not None else 0.0
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    code = _lib.DTYPE_F16 if query.dtype == torch.float16 else _lib.DTYPE_BF16
    null = ctypes.c_void_p(0)
    out = torch.empty((b, q_len, h, d), dtype=query.dtype, device=dev)
    for i in range(b):
        # q and the outputs hold the rows from token q_shift on: `pad` rows of padding, then the new tokens
        q_rows = torch.zeros((pad + q_len, h, d), dtype=query.dtype, device=dev)
        q_rows[pad:] = query[i].transpose(0, 1)
        out_rows = torch.empty((pad + q_len, h, d), dtype=query.dtype, device=dev)
        lse_rows = torch.empty((pad + q_len, h), dtype=torch.float32, device=dev)
        q_rows, k_rows, v_rows = E._in_place(q_rows, key[i].transpose(0, 1), value[i].transpose(0, 1))
        scratch = torch.empty(8 + 1 + m * h, dtype=torch.int32, device=dev)   # tile counters, then the redo list
        _lib.check(lib.moba_fwd_partials(
            E._ptr(q_rows), E._ptr(k_rows), E._ptr(v_rows), E._ptr(out_rows), E._ptr(lse_rows), null, null, null, null,
            at(0), at(2), null, at(4), at(4 + m), E._ptr(out_rows), E._ptr(lse_rows), kv_len, h, hkv, d, 0, 0, 1, kv_len,
            0, m, 1, E._strides(q_rows, k_rows), ctypes.c_void_p(scratch.data_ptr()),
            ctypes.c_void_p(scratch.data_ptr() + 32), scale, code, skip, q_shift, stream), "moba_fwd_partials")
        out[i] = out_rows[pad:]
    return out
