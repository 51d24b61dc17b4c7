"""Dense-mask MoBA on torch ops, registered as "moba_naive" like the reference's
educational implementation (moba/moba_naive.py:7-96).  It runs on whatever device
the tensors live on and is differentiable through autograd.  It is a separate
attention implementation for cross-checking small cases: "moba" never calls it.
"""

import math

import torch


def moba_attn_varlen_naive(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    moba_chunk_size: int,
    moba_topk: int,
) -> torch.Tensor:
    """Same arguments and result as moba/moba_naive.py:7-28: q, k, v [seqlen, heads, dim],
    returns [seqlen, heads, dim] in q's dtype.  Memory is O(heads * L^2) per sequence."""
    bounds = cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else list(cu_seqlens)
    B = int(moba_chunk_size)
    D = q.shape[-1]
    dev = q.device
    chunks_out = []
    for s0, s1 in zip(bounds[:-1], bounds[1:]):
        L = s1 - s0
        N = math.ceil(L / B)
        qs, ks, vs = q[s0:s1], k[s0:s1], v[s0:s1]
        pos = torch.arange(L, device=dev)
        chunk_of = pos // B                                        # [L]
        # chunk representatives, rounded to the input dtype as in moba_naive.py:43-50
        onehot = torch.nn.functional.one_hot(chunk_of, N).to(torch.float32)          # [L, N]
        reps = torch.einsum("ln,lhd->nhd", onehot, ks.float()) / onehot.sum(0)[:, None, None]
        reps = reps.to(k.dtype).float()
        score = torch.einsum("lhd,nhd->hln", qs.float(), reps)     # [H, L, N]
        cid = torch.arange(N, device=dev)
        score = torch.where(cid[None, :] > chunk_of[:, None], score.new_tensor(float("-inf")), score)
        score = torch.where(cid[None, :] == chunk_of[:, None], score.new_tensor(float("inf")), score)
        kk = min(int(moba_topk), N)
        vals, idx = torch.topk(score, kk, dim=-1, sorted=False)
        chosen = torch.zeros_like(score, dtype=torch.bool).scatter_(-1, idx, True)
        chosen &= score >= vals.amin(dim=-1, keepdim=True)
        visible = chosen[:, :, chunk_of] & (pos[:, None] >= pos[None, :])             # [H, L, L]
        logits = torch.einsum("xhd,yhd->hxy", qs.float(), ks.float()) * (D ** -0.5)
        prob = torch.softmax(logits.masked_fill(~visible, float("-inf")), dim=-1)
        chunks_out.append(torch.einsum("hxy,yhd->xhd", prob, vs.float()).to(q.dtype))
    return torch.cat(chunks_out, dim=0)
