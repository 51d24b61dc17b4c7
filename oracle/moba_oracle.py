"""CPU oracle for the MoBA attention path.

THIS FILE IS TEST INFRASTRUCTURE.  It is a torch-CPU / numpy restatement of the
reference algorithm, used only as the checker (tests, the smoke check, and the
``cpu_baseline`` leg of the benchmark).  The product never imports it.

Every function cites the reference lines whose behaviour it restates
(paths are relative to the reference checkout).

Pinned by (see tests/test_oracle_*.py):
  calc_chunks        hand-worked examples + brute-force loops
  chunk_mean         exact integer-valued inputs, torch ``float().mean()``
  gate_scores        torch einsum + brute-force mask loops
  select_topk        torch.topk sets on tie-free scores, full-sort brute force,
                     explicit tie cases for the tie rule stated below
  gather_lists       brute force + closed-form total count
  attend_dense       torch SDPA(is_causal) in the special cases that reduce to
                     it, uniform-V invariant, logsumexp of the attended set,
                     fp64 gradcheck
  merge_partials     closed form: merging a partition == attention over union
  moba_attn_varlen_naive
                     agreement with attend_dense(select_topk(...)) which is a
                     different formulation of the same attended set
No function here is "parity unpinned".
"""

from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------
# chunk metadata  (moba/moba_efficient.py:14-64)
# --------------------------------------------------------------------------
def calc_chunks(cu_seqlens: Sequence[int], chunk_size: int) -> dict:
    """Closed-form restatement of ``calc_chunks`` (moba/moba_efficient.py:14-64).

    Returns numpy arrays:
      cu_chunk[N+1]            token offset of every chunk start (:36-39)
      filtered_chunk_indices   global ids of chunks that are not the last chunk
                               of their sequence (:51-56)
      num_filtered_chunk       F (:57)
      chunk_to_batch[N]        sequence id of each chunk (:41-45)
    plus per-sequence helpers (n_chunks, first filtered id) used by the other
    oracle stages.
    """
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    assert cu.ndim == 1 and cu.size >= 2 and cu[0] == 0
    lens = np.diff(cu)
    assert (lens > 0).all(), "zero-length sequences are undefined in the reference"
    n_chunks = (lens + chunk_size - 1) // chunk_size
    cu_chunk = [0]
    chunk_to_batch = []
    filtered = []
    first_filtered = []
    cid = 0
    for b, (L, n) in enumerate(zip(lens, n_chunks)):
        first_filtered.append(len(filtered))
        for c in range(int(n)):
            size = min(chunk_size, int(L) - c * chunk_size)
            cu_chunk.append(cu_chunk[-1] + size)
            chunk_to_batch.append(b)
            if c != n - 1:
                filtered.append(cid)
            cid += 1
    return dict(
        cu_chunk=np.asarray(cu_chunk, dtype=np.int32),
        filtered_chunk_indices=np.asarray(filtered, dtype=np.int64),
        num_filtered_chunk=len(filtered),
        chunk_to_batch=np.asarray(chunk_to_batch, dtype=np.int32),
        n_chunks=n_chunks.astype(np.int64),
        first_filtered=np.asarray(first_filtered, dtype=np.int64),
        seq_lens=lens,
    )


def effective_topk(moba_topk: int, num_filtered_chunk: int) -> int:
    """k = min(moba_topk - 1, F)   (moba/moba_efficient.py:314)."""
    return min(moba_topk - 1, num_filtered_chunk)


# --------------------------------------------------------------------------
# key chunk-mean  (moba/moba_efficient.py:326-340 ; moba/moba_naive.py:43-50)
# --------------------------------------------------------------------------
def chunk_mean(k: torch.Tensor, cu_seqlens: Sequence[int], chunk_size: int) -> torch.Tensor:
    """Mean of K over every filtered (full) chunk, rounded to the input dtype.

    The reference takes ``.mean(dim=1)`` of a bf16 view and then ``.float()``
    (moba/moba_efficient.py:335-340): accumulate wide, round once to bf16.
    The oracle accumulates in fp64 (exact for any realistic bf16 data, hence
    independent of summation order), divides by B in fp64 and rounds that
    quotient once, to nearest-even, to the input dtype (through an fp32 value
    rounded to odd, so that the second rounding cannot land on the wrong side
    of a tie: ``round_once``).
    Returns [F, H, D] in k.dtype.
    """
    meta = calc_chunks(cu_seqlens, chunk_size)
    F = meta["num_filtered_chunk"]
    S, H, D = k.shape
    out = torch.empty((F, H, D), dtype=k.dtype)
    for i, cid in enumerate(meta["filtered_chunk_indices"]):
        s0 = int(meta["cu_chunk"][cid])
        blk = k[s0:s0 + chunk_size].to(torch.float64)
        assert blk.shape[0] == chunk_size
        mean64 = blk.sum(dim=0) / float(chunk_size)
        out[i] = round_once(mean64, k.dtype)
    return out


def round_once(x64: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """fp64 -> bf16/fp16 with a single round-to-nearest-even.  torch converts through fp32, and two nearest-even
    roundings in a row can differ from one (a value just above a tie of the narrow type that fp32 rounds onto
    the tie); rounding the intermediate fp32 to odd instead makes the second rounding see on which side of every
    tie the fp64 value lies."""
    f = x64.to(torch.float32)
    inexact = f.to(torch.float64) != x64
    away = f.to(torch.float64).abs() > x64.abs()
    u = f.view(torch.int32)
    u = torch.where(inexact & away, u - 1, u)      # the fp32 neighbour toward zero (bit patterns grow with |value|)
    u = torch.where(inexact, u | 1, u)
    return u.view(torch.float32).to(dtype)


# --------------------------------------------------------------------------
# gate scores + causal / sequence mask  (moba/moba_efficient.py:341-360)
# --------------------------------------------------------------------------
def gate_scores(q: torch.Tensor, kbar: torch.Tensor, cu_seqlens: Sequence[int],
                chunk_size: int) -> torch.Tensor:
    """fp32 gate[s, h, f] = <q[s,h,:], kbar[f,h,:]>, -inf where chunk f is not a
    valid history chunk of token s (moba/moba_efficient.py:345-360: masked when
    s < chunk_end[f] or s >= end of f's sequence).  Layout [S, H, F]."""
    meta = calc_chunks(cu_seqlens, chunk_size)
    S, H, D = q.shape
    F = meta["num_filtered_chunk"]
    gate = torch.einsum("shd,fhd->shf", q.float(), kbar.float())
    fidx = meta["filtered_chunk_indices"]
    chunk_end = meta["cu_chunk"][fidx + 1].astype(np.int64)
    batch_end = np.asarray(cu_seqlens, dtype=np.int64)[meta["chunk_to_batch"][fidx] + 1]
    s = np.arange(S, dtype=np.int64)[:, None]
    invalid = (s < chunk_end[None, :]) | (s >= batch_end[None, :])  # [S, F]
    gate.masked_fill_(torch.from_numpy(invalid)[:, None, :], NEG_INF)
    return gate


# --------------------------------------------------------------------------
# top-k selection  (moba/moba_efficient.py:362-371)
# --------------------------------------------------------------------------
def select_topk(gate: torch.Tensor, k: int) -> torch.Tensor:
    """Selected history chunks per (token, head).

    ``torch.topk(gate, k, dim=chunk)`` followed by dropping -inf picks
    (moba/moba_efficient.py:365-371).  The result is a set; this oracle returns
    it as int32 [S, H, k], ascending filtered-chunk ids, padded with -1.
    Tie rule (the reference inherits torch.topk's unspecified one): higher
    score first, then the lower chunk id.
    """
    S, H, F = gate.shape
    k = min(k, F)
    # stable descending sort keeps the lower index first among equal scores
    vals, idx = torch.sort(gate, dim=-1, descending=True, stable=True)
    vals, idx = vals[..., :k], idx[..., :k]
    idx = torch.where(torch.isinf(vals) & (vals < 0), torch.full_like(idx, F + 1), idx)
    idx, _ = torch.sort(idx, dim=-1)
    idx = torch.where(idx > F, torch.full_like(idx, -1), idx)
    return idx.to(torch.int32)


def selection_mask(sel: torch.Tensor, F: int) -> torch.Tensor:
    """bool [F, H, S] view of a selection (the reference's ``gate_mask``,
    moba/moba_efficient.py:367-371)."""
    S, H, K = sel.shape
    m = torch.zeros((S, H, F + 1), dtype=torch.bool)
    m.scatter_(2, torch.where(sel < 0, torch.full_like(sel, F), sel).long(), True)
    return m[..., :F].permute(2, 1, 0).contiguous()


# --------------------------------------------------------------------------
# varlen gather lists  (moba/moba_efficient.py:373-386)
# --------------------------------------------------------------------------
def gather_lists(sel: torch.Tensor, F: int):
    """Brute-force index lists in the reference's order: filtered chunk major,
    then head, then token ascending (moba/moba_efficient.py:375-379).

    Returns (seg_count[F*H], seg_offset[F*H+1], rows[M], slots[M]) where rows is
    the token index and slots the position j of that chunk inside sel[s,h,:].
    """
    S, H, K = sel.shape
    sel_np = sel.numpy()
    counts = np.zeros(F * H, dtype=np.int64)
    rows, slots = [], []
    for f in range(F):
        for h in range(H):
            hit = np.argwhere(sel_np[:, h, :] == f)  # sorted by token (then slot)
            counts[f * H + h] = hit.shape[0]
            rows.extend(hit[:, 0].tolist())
            slots.extend(hit[:, 1].tolist())
    offs = np.concatenate([[0], np.cumsum(counts)])
    return counts, offs, np.asarray(rows, dtype=np.int64), np.asarray(slots, dtype=np.int64)


def expected_pair_count(cu_seqlens: Sequence[int], chunk_size: int, k: int, H: int) -> int:
    """M = H * sum_b sum_c |chunk c| * min(k, c): the number of selected
    (token, head, history chunk) triples is data independent, because a token in
    the c-th chunk of its sequence has exactly c valid candidates
    (moba/moba_efficient.py:355-371)."""
    meta = calc_chunks(cu_seqlens, chunk_size)
    total = 0
    for L, n in zip(meta["seq_lens"], meta["n_chunks"]):
        for c in range(int(n)):
            size = min(chunk_size, int(L) - c * chunk_size)
            total += size * min(k, c)
    return total * H


def attention_flops(cu_seqlens: Sequence[int], chunk_size: int, moba_topk: int, H: int, D: int) -> float:
    """Forward FLOPs actually required: 4*D per attended (query, key) pair."""
    meta = calc_chunks(cu_seqlens, chunk_size)
    k = effective_topk(moba_topk, meta["num_filtered_chunk"])
    pairs = 0
    if k <= 0:
        for L in meta["seq_lens"]:
            pairs += int(L) * (int(L) + 1) // 2
        return 4.0 * D * H * pairs
    for L, n in zip(meta["seq_lens"], meta["n_chunks"]):
        for c in range(int(n)):
            size = min(chunk_size, int(L) - c * chunk_size)
            pairs += size * (size + 1) // 2 + size * min(k, c) * chunk_size
    return 4.0 * D * H * pairs


# --------------------------------------------------------------------------
# attention over the attended set  (moba/moba_naive.py:76-94, moba_efficient.py:86)
# --------------------------------------------------------------------------
def attended_mask(sel: Optional[torch.Tensor], cu_seqlens: Sequence[int], chunk_size: int,
                  b: int, H: int) -> torch.Tensor:
    """bool [H, L, L] for sequence b: key u is attended by query t iff u is in
    t's own chunk and u <= t, or u lies in a selected history chunk.
    ``sel is None`` means full causal attention (the k <= 0 fallback,
    moba/moba_efficient.py:318-321)."""
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    s0, s1 = int(cu[b]), int(cu[b + 1])
    L = s1 - s0
    t = torch.arange(L)
    causal = t[:, None] >= t[None, :]
    if sel is None:
        return causal[None].expand(H, L, L).clone()
    meta = calc_chunks(cu_seqlens, chunk_size)
    fb = int(meta["first_filtered"][b])
    qc = t // chunk_size
    kc = t // chunk_size
    own = (qc[:, None] == kc[None, :]) & causal                       # [L, L]
    sel_b = sel[s0:s1].long() - fb                                      # local chunk ids, <0 = none
    n = int(meta["n_chunks"][b])
    chunk_sel = torch.zeros((L, H, n + 1), dtype=torch.bool)
    chunk_sel.scatter_(2, torch.where(sel[s0:s1] < 0, torch.full_like(sel_b, n), sel_b), True)
    chunk_sel = chunk_sel[..., :n]                                      # [L, H, n]
    hist = chunk_sel[:, :, kc]                                          # [L, H, L]
    return own[None] | hist.permute(1, 0, 2)


def attend_dense(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: Sequence[int],
                 chunk_size: int, sel: Optional[torch.Tensor], dtype=torch.float32,
                 return_lse: bool = False):
    """softmax(D^-1/2 q k^T restricted to the attended set) v in ``dtype`` math
    (fp32 like moba/moba_naive.py:84-94; scale D^-0.5 per moba_efficient.py:86).
    Differentiable with respect to q, k, v; the selection is a constant
    (moba/moba_efficient.py:365 discards the top-k values).
    Returns [S, H, D] in ``dtype`` (and the natural-log LSE [S, H])."""
    S, H, D = q.shape
    scale = D ** -0.5
    outs, lses = [], []
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    for b in range(cu.size - 1):
        s0, s1 = int(cu[b]), int(cu[b + 1])
        mask = attended_mask(sel, cu_seqlens, chunk_size, b, H)
        qf, kf, vf = (x[s0:s1].to(dtype) for x in (q, k, v))
        logits = torch.einsum("xhd,yhd->hxy", qf, kf) * scale
        logits = logits.masked_fill(~mask, NEG_INF)
        lse = torch.logsumexp(logits, dim=-1)                            # [H, L]
        p = torch.exp(logits - lse[..., None])
        outs.append(torch.einsum("hxy,yhd->xhd", p, vf))
        lses.append(lse.t())
    out = torch.cat(outs, dim=0)
    if return_lse:
        return out, torch.cat(lses, dim=0)
    return out


# --------------------------------------------------------------------------
# whole operator with the efficient path's semantics  (moba_efficient.py:270-443)
# --------------------------------------------------------------------------
def moba_attn_varlen_oracle(q, k, v, cu_seqlens: Sequence[int], max_seqlen: int, moba_chunk_size: int,
                            moba_topk: int, sel: Optional[torch.Tensor] = None, return_aux: bool = False):
    """fp32 oracle of ``moba_attn_varlen`` (moba/moba_efficient.py:270-443),
    including the k <= 0 fallback to full causal attention (:313-321).
    If ``sel`` is given it replaces the oracle's own selection (used to check the
    attention stage on the kernel's selection so that near-tie flips of the gate do
    not masquerade as attention errors)."""
    meta = calc_chunks(cu_seqlens, moba_chunk_size)
    keff = effective_topk(moba_topk, meta["num_filtered_chunk"])
    if keff <= 0:
        out, lse = attend_dense(q, k, v, cu_seqlens, moba_chunk_size, None, return_lse=True)
        return (out, lse, None) if return_aux else out
    if sel is None:
        kbar = chunk_mean(k.detach(), cu_seqlens, moba_chunk_size)
        gate = gate_scores(q.detach(), kbar, cu_seqlens, moba_chunk_size)
        sel = select_topk(gate, keff)
    out, lse = attend_dense(q, k, v, cu_seqlens, moba_chunk_size, sel, return_lse=True)
    return (out, lse, sel) if return_aux else out


# --------------------------------------------------------------------------
# LSE merge of partial attentions  (moba/moba_efficient.py:119-168)
# --------------------------------------------------------------------------
def merge_partials(outs: torch.Tensor, lses: torch.Tensor):
    """Combine partial attentions over disjoint key sets.
    outs [P, ..., D] are per-part normalised outputs, lses [P, ...] their natural
    log-sum-exp (-inf for an empty part).  Algebra of moba_efficient.py:130-168:
    LSE = log sum_p exp(lse_p);  out = sum_p out_p * exp(lse_p - LSE)."""
    lse = torch.logsumexp(lses, dim=0)
    w = torch.exp(lses - lse[None])
    w = torch.where(torch.isinf(lses) & (lses < 0), torch.zeros_like(w), w)
    out = (torch.where(w[..., None] == 0, torch.zeros_like(outs), outs) * w[..., None]).sum(dim=0)
    return out, lse


# --------------------------------------------------------------------------
# the dense-mask formulation of moba/moba_naive.py:29-96  (also the CPU baseline)
# --------------------------------------------------------------------------
def moba_attn_varlen_naive(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens, max_seqlen: int,
                           moba_chunk_size: int, moba_topk: int) -> torch.Tensor:
    """Restatement of ``moba_attn_varlen_naive`` (moba/moba_naive.py:7-96).

    Per sequence (:34): chunk representatives incl. the partial last chunk
    (:43-50), fp32 gate over the sequence's own chunks (:53-55), a token's own
    chunk forced in with +inf and chunks not strictly in its past removed with
    -inf (:58-61), top-min(topk, N) along chunks (:63-65), membership by value
    threshold AND index (:66-73), expansion chunk->token and a causal cut
    (:76-81), fp32 softmax(scale * (q k^T + 0/-inf)) v (:84-94).
    Note the topk=1 behaviour (own chunk only) differs from the efficient path.
    """
    cu = [int(x) for x in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    S, H, D = q.shape
    B = moba_chunk_size
    scale = D ** -0.5
    pieces = []
    for b in range(len(cu) - 1):
        s0, s1 = cu[b], cu[b + 1]
        L = s1 - s0
        N = math.ceil(L / B)
        qb, kb, vb = q[s0:s1], k[s0:s1], v[s0:s1]
        reps = torch.stack([kb[c * B:min(L, (c + 1) * B)].mean(dim=0) for c in range(N)], dim=0)  # [N,H,D] in k dtype
        gate = torch.einsum("shd,nhd->hsn", qb.float(), reps.float())                               # [H,L,N]
        tok_chunk = torch.arange(L) // B                                                            # [L]
        cidx = torch.arange(N)
        future = cidx[None, :] > tok_chunk[:, None]                                                 # chunk after the token's
        own = cidx[None, :] == tok_chunk[:, None]
        gate = gate.masked_fill(future[None], NEG_INF).masked_fill(own[None], float("inf"))
        kk = min(moba_topk, N)
        top_val, top_idx = torch.topk(gate, k=kk, dim=-1, largest=True, sorted=False)
        thresh = top_val.min(dim=-1, keepdim=True).values
        picked = torch.zeros_like(gate, dtype=torch.bool).scatter_(-1, top_idx, True)
        keep = picked & (gate >= thresh)                                                            # [H,L,N]
        keep_tok = keep[:, :, tok_chunk]                                                            # [H,L,L]
        causal = torch.arange(L)[:, None] >= torch.arange(L)[None, :]
        allow = keep_tok & causal[None]
        logits = torch.einsum("xhd,yhd->hxy", qb.float(), kb.float())
        logits = torch.where(allow, logits, torch.full_like(logits, NEG_INF)) * scale
        p = logits.softmax(dim=-1)
        pieces.append(torch.einsum("hxy,yhd->xhd", p, vb.float()).to(q.dtype))
    return torch.cat(pieces, dim=0)


# --------------------------------------------------------------------------
# blocked formulation for sizes where [H, L, L] does not fit  (same set semantics)
# --------------------------------------------------------------------------
def attend_blocked(q, k, v, cu_seqlens: Sequence[int], chunk_size: int, sel: Optional[torch.Tensor],
                   rows: Optional[np.ndarray] = None):
    """Attention over the attended set for a subset of token rows, one row block
    at a time (no L x L tensor).  Same semantics as ``attend_dense``; used to
    spot-check large configurations on sampled rows.  Returns (out[R,H,D] fp32,
    lse[R,H] fp32) for the given global token indices (default: all)."""
    S, H, D = q.shape
    scale = D ** -0.5
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    meta = calc_chunks(cu_seqlens, chunk_size)
    if rows is None:
        rows = np.arange(S)
    out = torch.zeros((len(rows), H, D), dtype=torch.float32)
    lse = torch.zeros((len(rows), H), dtype=torch.float32)
    for i, s in enumerate(rows):
        b = int(np.searchsorted(cu, s, side="right") - 1)
        s0 = int(cu[b])
        t = int(s) - s0
        c = t // chunk_size
        fb = int(meta["first_filtered"][b])
        for h in range(H):
            keys = list(range(s0 + c * chunk_size, int(s) + 1))
            if sel is None:
                keys = list(range(s0, int(s) + 1))
            else:
                for f in sel[s, h].tolist():
                    if f >= 0:
                        lc = f - fb
                        keys.extend(range(s0 + lc * chunk_size, s0 + (lc + 1) * chunk_size))
            kk = k[keys, h].float()
            logits = (kk @ q[s, h].float()) * scale
            l = torch.logsumexp(logits, dim=0)
            out[i, h] = torch.exp(logits - l) @ v[keys, h].float()
            lse[i, h] = l
    return out, lse
