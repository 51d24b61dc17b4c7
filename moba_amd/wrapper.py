"""transformers attention-interface adapter, mirroring moba/wrapper.py:29-84.

Prefill (q_len == kv_len) converts the HF layout [batch, heads, seq, dim] to the packed
varlen layout and calls the MoBA operator (KV heads are expanded to the query heads first
unless the operator handles grouped-query attention itself).
Decode (q_len != kv_len) is full causal attention over the KV cache, as in the
reference (moba/wrapper.py:76-82): the HIP decode kernel for one new token with the "moba"
implementation, PyTorch's scaled_dot_product_attention otherwise.
"""

from typing import Callable, Optional, Tuple

import torch
import torch.nn.functional as F

from .config import MoBAConfig


_CU_SEQLENS = {}  # (batch, seq_len, device) -> int32 tensor of multiples of seq_len


def _cu_seqlens_for(batch: int, seq_len: int, device) -> torch.Tensor:
    """cu_seqlens of `batch` sequences of `seq_len` tokens; one tensor per shape, so that an operator
    which remembers the batch layout per tensor recognises it on every layer and step."""
    key = (batch, seq_len, str(device))
    t = _CU_SEQLENS.get(key)
    if t is None:
        if len(_CU_SEQLENS) >= 16:
            _CU_SEQLENS.pop(next(iter(_CU_SEQLENS)))
        # Made outside inference mode even when the model runs inside it: an inference tensor has no version
        # counter, the planner would not remember it by identity, and every layer would then read it back from
        # the device (a blocking copy) to plan by value.  Nobody writes to this tensor.
        with torch.inference_mode(False):
            t = torch.arange(0, (batch + 1) * seq_len, seq_len, dtype=torch.int32, device=device)
        _CU_SEQLENS[key] = t
    return t


def _hip_decode(moba_impl, query, key, value, several=False) -> bool:
    """The HIP decode kernels serve the HIP operator's registrations ("moba"), for the shapes they support;
    anything else decodes with PyTorch's scaled_dot_product_attention."""
    if not getattr(moba_impl, "takes_host_lengths", False):
        return False
    from .decode import chunk_supported, supported
    return chunk_supported(query, key, value) if several else supported(query, key, value)


def hf_to_fa(x: torch.Tensor) -> torch.Tensor:
    """[batch, heads, seqlen, head_dim] -> [batch * seqlen, heads, head_dim] (moba/wrapper.py:7-15)."""
    b, h, s, d = x.shape
    return x.transpose(1, 2).reshape(b * s, h, d)


def fa_to_hf(x: torch.Tensor, batch: int) -> torch.Tensor:
    """[batch * seqlen, heads, head_dim] -> [batch, heads, seqlen, head_dim] (moba/wrapper.py:18-26)."""
    return x.view(batch, -1, x.shape[1], x.shape[2]).transpose(1, 2)


def moba_layer(
    moba_impl: Callable,
    moba_config: MoBAConfig,
    module: torch.nn.Module,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    *args,
    dropout: float = 0.0,
    scaling: Optional[float] = None,
    **kwargs,
) -> Tuple[torch.Tensor, None]:
    """
    Args:
        query: [batch, q_heads, q_len, head_dim]
        key, value: [batch, kv_heads, kv_len, head_dim]
    Returns:
        (attn_output, None); prefill output is [batch * q_len, q_heads, head_dim], which the
        caller's reshape(batch, q_len, -1) absorbs exactly as with the reference
        (moba/wrapper.py:83 leaves the conversion back commented out).
    """
    assert module.is_causal
    batch, q_heads, q_len, head_dim = query.shape
    _, kv_heads, kv_len, _ = key.shape
    if q_len == kv_len:
        chunk_size = moba_config.moba_chunk_size
        num_layers = getattr(getattr(module, "config", None), "num_hidden_layers", None)
        if moba_config.is_full_attention_layer(getattr(module, "layer_idx", None), num_layers):
            # one chunk per sequence: no history chunks, and every implementation of the operator then
            # computes plain causal attention (moba/moba_efficient.py:313-321, moba/moba_naive.py:58-81)
            chunk_size = max(chunk_size, kv_len)
        batched = getattr(moba_impl, "batched_impl", None) if batch > 1 else None
        if batched is not None:
            # an implementation that reads [batch, heads, seqlen, head_dim] in place (the HIP operator): no
            # transposing copies of q, k, v (hf_to_fa's reshape copies when batch > 1, moba/wrapper.py:56-58)
            # and no key/value head expansion
            return batched(query, key, value, chunk_size, moba_config.moba_topk), None
        q = hf_to_fa(query)
        k = hf_to_fa(key)
        v = hf_to_fa(value)
        rep = q_heads // kv_heads
        if rep > 1:
            # an implementation that indexes key/value heads itself (the HIP operator) takes them as they are;
            # others get the expanded copies, as in the reference (moba/wrapper.py:59-61)
            grouped = getattr(moba_impl, "grouped_query_impl", None)
            if grouped is not None:
                moba_impl = grouped
            else:
                k = torch.repeat_interleave(k, rep, dim=1)
                v = torch.repeat_interleave(v, rep, dim=1)
        cu_seqlens = _cu_seqlens_for(batch, kv_len, query.device)
        if getattr(moba_impl, "takes_host_lengths", False):
            # the lengths are known here on the host: spare the operator its device-to-host read
            from .plan import make_plan
            make_plan(cu_seqlens, chunk_size, moba_config.moba_topk,
                      host_lengths=range(0, (batch + 1) * kv_len, kv_len))
        out = moba_impl(
            q=q,
            k=k,
            v=v,
            cu_seqlens=cu_seqlens,
            max_seqlen=kv_len,
            moba_chunk_size=chunk_size,
            moba_topk=moba_config.moba_topk,
        )
    elif q_len == 1 and dropout == 0.0 and _hip_decode(moba_impl, query, key, value):
        # one new token against the cache: the HIP decode kernel reads K and V once, in place
        from .decode import decode_attention
        out = decode_attention(query, key, value, scaling)
    elif q_len < kv_len and dropout == 0.0 and _hip_decode(moba_impl, query, key, value, several=True):
        # several new tokens against the cache: the decode kernel per token, or the forward kernel's causal tiles
        from .decode import chunk_decode_attention
        out = chunk_decode_attention(query, key, value, scaling)
    else:
        # decode: every cached key is visible to the new queries (bottom-right aligned causal mask)
        mask = None
        if q_len > 1:
            qi = torch.arange(q_len, device=query.device)[:, None] + (kv_len - q_len)
            mask = torch.arange(kv_len, device=query.device)[None, :] <= qi
        out = F.scaled_dot_product_attention(query, key, value, attn_mask=mask, dropout_p=dropout, scale=scaling,
                                             enable_gqa=q_heads != kv_heads)
        out = out.transpose(1, 2)
    return out, None
