"""Chunk metadata of a packed batch, computed on the host from ``cu_seqlens``.

Counterpart of ``calc_chunks`` (moba/moba_efficient.py:14-64) plus everything else
that depends only on the sequence lengths: buffer sizes, tile counts and the small
int32 tables the kernels index.  All sizes are data independent (a token in the c-th
chunk of its sequence selects exactly min(k, c) history chunks), so one device-to-host
read of ``cu_seqlens`` is the only synchronisation of a forward call, and a caller that
knows the lengths on the host (the transformers adapter does) avoids even that.
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import numpy as np
import torch

TILE_ROWS = 128      # query rows per workgroup of the backward kernels
FWD_TILE_ROWS = 256  # ... and of the forward kernel


@dataclass
class MobaPlan:
    cu: List[int]
    chunk_size: int
    moba_topk: int
    S: int
    nseq: int
    N: int              # chunks
    F: int              # filtered chunks (possible history chunks)
    k_eff: int          # min(moba_topk - 1, F)   (moba/moba_efficient.py:314)
    K: int              # slots per (token, head): min(k_eff, most history chunks any token has)
    fallback: bool      # k_eff <= 0: full causal attention (moba/moba_efficient.py:318-321)
    P: int              # (filtered chunk, later chunk of the same sequence) pairs
    cmax: int           # max chunks per sequence minus one
    pairs_per_head: int  # list entries per head (M / H): selected (token, chunk) pairs of the tokens beyond the dense prefixes
    self_tiles: int     # row tiles of the attention chunks, per head (TILE_ROWS rows each; tables self_tile_*)
    fwd_self_tiles: int  # the same in tiles of FWD_TILE_ROWS rows (tables fwd_self_tile_*)
    flops_per_head: float
    # Dense prefixes.  A token in chunk c <= K of its sequence selects every earlier chunk, so what it attends is
    # the plain causal prefix.  With dense_local = d (0 <= d <= K) the chunks 0..d of every sequence form one
    # attention chunk whose rows run through the causal self path alone: no gate, no list entries and one partial
    # result for them.  d = 0 is the reference's own decomposition (every chunk its own attention chunk).
    dense_local: int = 0
    NA: int = 0         # attention chunks (tables achunk_tok, self_tile_*, fwd_self_tile_*)
    kv_tiles: int = 0   # key tiles of TILE_ROWS keys of the chunks, per key/value head (tables kv_tile_*)
    # The rows of a sequence's first attention chunk have no history slots: the forward kernel writes them straight
    # to the output (table achunk_direct) and the merge walks the other tokens only (tables mrg_start, mrg_prefix).
    merge_tokens: int = 0
    tables: Dict[str, torch.Tensor] = field(default_factory=dict)
    host: Dict[str, np.ndarray] = field(default_factory=dict)
    memo: Dict[tuple, object] = field(default_factory=dict)  # what callers derive once per plan (sizes, pointers)
    device: object = None

    def hist_tile_bound(self, H: int, rows: int = TILE_ROWS) -> int:
        """Upper bound on the number of history tiles of `rows` rows (every segment may end in a partial tile)."""
        return (self.pairs_per_head * H) // rows + self.F * H

    def with_dense_prefix(self) -> "MobaPlan":
        """The plan of the same batch with the first K + 1 chunks of every sequence as one attention chunk."""
        if self.fallback or self.dense_local == self.K:
            return self
        return _build(np.asarray(self.cu, dtype=np.int64), self.chunk_size, self.moba_topk, self.device, dense=True)


def _host_tables(cu: np.ndarray, B: int, topk: int, dense: bool = False):
    lens = np.diff(cu)
    nseq = lens.size
    n_chunks = (lens + B - 1) // B
    F = int((n_chunks - 1).sum())
    k_eff = min(topk - 1, F)
    fallback = k_eff <= 0
    if fallback:
        # one "chunk" per sequence: the self part alone is full causal attention
        n_chunks = np.ones_like(n_chunks)
        chunk_tok = cu.copy()
        chunk_len = lens
        seq_of_chunk = np.arange(nseq)
        local = np.zeros(nseq, dtype=np.int64)
        K = d = 0
    else:
        seq_of_chunk = np.repeat(np.arange(nseq), n_chunks)
        cbase = np.concatenate([[0], np.cumsum(n_chunks)])[:-1]
        local = np.arange(int(n_chunks.sum())) - cbase[seq_of_chunk]
        chunk_start = cu[seq_of_chunk] + local * B
        chunk_len = np.minimum(B, cu[seq_of_chunk + 1] - chunk_start)
        chunk_tok = np.concatenate([chunk_start, [cu[-1]]])
        cmax = int(n_chunks.max() - 1)
        K = min(k_eff, cmax)
        d = K if dense else 0
    N = int(n_chunks.sum())
    # attention chunks: chunks 0..d of a sequence together, every later chunk alone
    starts_a = (local == 0) | (local > d)
    achunk_tok = np.concatenate([chunk_tok[:-1][starts_a], [cu[-1]]])
    achunk_len = np.diff(achunk_tok)
    NA = achunk_len.size
    achunk_of = np.cumsum(starts_a) - 1                      # attention chunk of every chunk
    tiles = (achunk_len + TILE_ROWS - 1) // TILE_ROWS
    ftiles = (achunk_len + FWD_TILE_ROWS - 1) // FWD_TILE_ROWS
    ktiles = (chunk_len + TILE_ROWS - 1) // TILE_ROWS
    out = dict(chunk_tok=chunk_tok, achunk_tok=achunk_tok,
               fwd_self_tile_prefix=np.concatenate([[0], np.cumsum(ftiles)]),
               fwd_self_tile_chunk=np.repeat(np.arange(NA), ftiles),
               self_tile_prefix=np.concatenate([[0], np.cumsum(tiles)]),
               self_tile_chunk=np.repeat(np.arange(NA), tiles),
               kv_tile_prefix=np.concatenate([[0], np.cumsum(ktiles)]),
               kv_tile_chunk=np.repeat(np.arange(N), ktiles),
               chunk_self_end=achunk_tok[achunk_of + 1],     # where the causal rows of a chunk's keys end
               achunk_direct=(local[starts_a] == 0).astype(np.int64))
    # the tokens behind the first attention chunk of every sequence: ranges of the merge
    first_end = achunk_tok[1:][local[starts_a] == 0]         # end of the first attention chunk of every sequence
    out.update(mrg_start=first_end, mrg_prefix=np.concatenate([[0], np.cumsum(cu[1:] - first_end)]))
    info = dict(nseq=nseq, N=N, F=0 if fallback else F, k_eff=k_eff, fallback=fallback, K=0, P=0, cmax=0,
                pairs_per_head=0, self_tiles=int(tiles.sum()), fwd_self_tiles=int(ftiles.sum()), NA=NA, dense_local=d,
                kv_tiles=int(ktiles.sum()), merge_tokens=int((cu[1:] - first_end).sum()))
    pairs_self = int((chunk_len.astype(np.int64) * (chunk_len + 1) // 2).sum())
    if not fallback:
        seq_fbase = np.concatenate([[0], np.cumsum(n_chunks - 1)])
        is_last = local == n_chunks[seq_of_chunk] - 1
        fidx = np.nonzero(~is_last)[0]
        fchunk_tok = chunk_start[fidx]
        nq = (n_chunks[seq_of_chunk] - 1 - local)[fidx]          # later chunks of the same sequence
        pair_off = np.concatenate([[0], np.cumsum(nq)])
        pairs_all = int((chunk_len.astype(np.int64) * np.minimum(K, local)).sum())
        pairs = int((chunk_len.astype(np.int64) * np.where(local > d, np.minimum(K, local), 0)).sum())
        chunk_fid = np.full(N, -1, dtype=np.int64)
        chunk_fid[fidx] = np.arange(F)
        out.update(seq_fbase=seq_fbase, fchunk_tok=fchunk_tok, chunk_fb=seq_fbase[seq_of_chunk], chunk_local=local,
                   pair_off=pair_off, chunk_fid=chunk_fid)
        info.update(K=K, P=int(nq.sum()), cmax=cmax, pairs_per_head=pairs)
        flops = 4.0 * (pairs_self + pairs_all * B)
    else:
        flops = 4.0 * pairs_self
    info["flops_per_head_per_d"] = flops
    return out, info


# Plans are cached two ways.  By value: (lengths, chunk size, top-k, device) -> plan, so equal
# batches share tables whatever tensor describes them.  By tensor: (id, version) of a device
# cu_seqlens tensor -> plan, which saves the device-to-host read on later calls; the entry keeps the
# tensor alive, so its id cannot be reused by another tensor while the entry exists (the reference
# memoises on tensor identity too, moba/moba_efficient.py:14, and is stale after an in-place update;
# the version number closes that hole here).
_BY_VALUE: "OrderedDict[Tuple, MobaPlan]" = OrderedDict()
_BY_TENSOR: "OrderedDict[Tuple, Tuple[MobaPlan, torch.Tensor]]" = OrderedDict()
_CACHE_SIZE = 16


def _remember(cache, key, value):
    cache[key] = value
    cache.move_to_end(key)
    while len(cache) > _CACHE_SIZE:
        cache.popitem(last=False)


def _build(cu: np.ndarray, chunk_size: int, moba_topk: int, device, dense: bool = False) -> MobaPlan:
    if cu.ndim != 1 or cu.size < 2:
        raise ValueError("cu_seqlens must be a 1-D tensor with at least two entries")
    if cu[0] != 0 or (np.diff(cu) <= 0).any():
        raise ValueError("cu_seqlens must start at 0 and be strictly increasing (zero-length sequences are unsupported)")
    if chunk_size <= 0 or moba_topk <= 0:
        raise ValueError("moba_chunk_size and moba_topk must be positive")
    on_device = device is not None and torch.device(device).type != "cpu"
    vkey = (cu.tobytes(), int(chunk_size), int(moba_topk), str(device) if on_device else None, bool(dense))
    hit = _BY_VALUE.get(vkey)
    if hit is not None:
        _BY_VALUE.move_to_end(vkey)
        return hit
    host, info = _host_tables(cu, int(chunk_size), int(moba_topk), dense)
    host["cu_seqlens"] = cu  # the kernels read the plan's own copy, never the caller's tensor
    plan = MobaPlan(cu=cu.tolist(), chunk_size=int(chunk_size), moba_topk=int(moba_topk), S=int(cu[-1]),
                    nseq=info["nseq"], N=info["N"], F=info["F"], k_eff=info["k_eff"], K=info["K"],
                    fallback=info["fallback"], P=info["P"], cmax=info["cmax"], pairs_per_head=info["pairs_per_head"],
                    self_tiles=info["self_tiles"], fwd_self_tiles=info["fwd_self_tiles"],
                    flops_per_head=info["flops_per_head_per_d"], dense_local=info["dense_local"], NA=info["NA"],
                    kv_tiles=info["kv_tiles"], merge_tokens=info["merge_tokens"], host=host,
                    device=device if on_device else None)
    if on_device:
        names = list(host)
        flat = np.concatenate([host[n_].astype(np.int32) for n_ in names])
        dev = torch.from_numpy(flat).to(device)
        off = 0
        for n_ in names:
            plan.tables[n_] = dev[off:off + host[n_].size]
            off += host[n_].size
    _remember(_BY_VALUE, vkey, plan)
    return plan


def make_plan(cu_seqlens, chunk_size: int, moba_topk: int, device=None, host_lengths=None) -> MobaPlan:
    """Build (or fetch) the plan for a batch.  ``cu_seqlens`` may be a device tensor (read once, then
    remembered for that tensor and version) or a Python sequence.  ``host_lengths`` is an optional host
    copy of a device ``cu_seqlens`` supplied by a caller that built it: no device-to-host read happens."""
    if not torch.is_tensor(cu_seqlens):
        return _build(np.asarray(list(cu_seqlens), dtype=np.int64), chunk_size, moba_topk, device)
    device = cu_seqlens.device if device is None else device
    # An inference tensor (made under torch.inference_mode()) has no version counter, so an in-place update
    # could not be noticed: such a tensor is never remembered by identity.  It costs one small device-to-host
    # read per call unless the caller supplies host_lengths (the transformers adapter does).
    if cu_seqlens.is_inference():
        if host_lengths is not None:
            cu = np.asarray(list(host_lengths), dtype=np.int64)
        else:
            cu = cu_seqlens.detach().to("cpu", torch.int64).numpy()
        return _build(cu, chunk_size, moba_topk, device)
    tkey = (id(cu_seqlens), cu_seqlens._version, str(device), int(chunk_size), int(moba_topk))
    hit = _BY_TENSOR.get(tkey)
    if hit is not None and hit[1] is cu_seqlens:
        _BY_TENSOR.move_to_end(tkey)
        return hit[0]
    if host_lengths is not None:
        cu = np.asarray(list(host_lengths), dtype=np.int64)
    else:
        cu = cu_seqlens.detach().to("cpu", torch.int64).numpy()
    plan = _build(cu, chunk_size, moba_topk, device)
    _remember(_BY_TENSOR, tkey, (plan, cu_seqlens))
    return plan
