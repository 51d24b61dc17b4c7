"""Decode attention kernel (one query token against the key/value cache) against an fp32
softmax on the same inputs; through the C ABI, and through the adapter's decode branch."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref(q, k, v, scale):
    rep = q.shape[1] // k.shape[1]
    kk = k.float().repeat_interleave(rep, dim=1)
    vv = v.float().repeat_interleave(rep, dim=1)
    p = torch.softmax((q.float() @ kk.transpose(-1, -2)) * scale, dim=-1)
    return (p @ vv).transpose(1, 2)            # [B, 1, H, D]


@pytest.mark.parametrize("B,H,Hkv,Skv,dtype", [
    (1, 32, 8, 131072, torch.bfloat16),
    (2, 8, 8, 1000, torch.bfloat16),
    (3, 16, 2, 4097, torch.float16),
    (1, 4, 2, 1, torch.bfloat16),
    (5, 2, 1, 37, torch.float16),
    (4, 32, 8, 777, torch.bfloat16),
])
def test_decode_matches_softmax(B, H, Hkv, Skv, dtype):
    from moba_amd.decode import decode_attention
    print("decode case", B, H, Hkv, Skv, dtype, flush=True)
    g = torch.Generator(device="cuda").manual_seed(Skv)
    q = torch.randn((B, H, 1, 128), generator=g, device="cuda").to(dtype)
    k = torch.randn((B, Hkv, Skv, 128), generator=g, device="cuda").to(dtype)
    v = torch.randn((B, Hkv, Skv, 128), generator=g, device="cuda").to(dtype)
    for scale in (None, 0.2):
        out = decode_attention(q, k, v, scale)
        want = _ref(q, k, v, 128 ** -0.5 if scale is None else scale)
        assert out.shape == (B, 1, H, 128)
        err = (out.float() - want).abs()
        assert err.max() < 1e-2 and err.mean() < 1e-3, (err.max().item(), err.mean().item())


def test_decode_reads_a_cache_view_in_place():
    """A preallocated cache [B, Hkv, Smax, D] sliced to the filled length: strided, not copied."""
    from moba_amd.decode import decode_attention
    g = torch.Generator(device="cuda").manual_seed(1)
    cache_k = torch.randn((2, 4, 512, 128), generator=g, device="cuda").to(torch.bfloat16)
    cache_v = torch.randn((2, 4, 512, 128), generator=g, device="cuda").to(torch.bfloat16)
    q = torch.randn((2, 8, 1, 128), generator=g, device="cuda").to(torch.bfloat16)
    k, v = cache_k[:, :, :300], cache_v[:, :, :300]
    assert not k.is_contiguous()
    out = decode_attention(q, k, v)
    err = (out.float() - _ref(q, k, v, 128 ** -0.5)).abs()
    assert err.max() < 1e-2


def test_adapter_decode_branch_uses_the_kernel_and_agrees_with_sdpa():
    from moba_amd import MoBAConfig, moba_attn_varlen
    from moba_amd.moba_naive import moba_attn_varlen_naive
    from moba_amd.wrapper import moba_layer

    class Mod(torch.nn.Module):
        is_causal = True

    g = torch.Generator(device="cuda").manual_seed(2)
    q = torch.randn((2, 8, 1, 128), generator=g, device="cuda").to(torch.bfloat16)
    k = torch.randn((2, 2, 333, 128), generator=g, device="cuda").to(torch.bfloat16)
    v = torch.randn((2, 2, 333, 128), generator=g, device="cuda").to(torch.bfloat16)
    cfg = MoBAConfig(64, 3)
    a, _ = moba_layer(moba_attn_varlen, cfg, Mod(), q, k, v, None)          # HIP decode kernel
    b, _ = moba_layer(moba_attn_varlen_naive, cfg, Mod(), q, k, v, None)    # SDPA
    assert a.shape == b.shape == (2, 1, 8, 128)
    assert (a.float() - b.float()).abs().max() < 2e-2


def _ref_tail(q, k, v, scale):
    """fp32 attention of the last q_len tokens: token j sees the keys up to position Skv - q_len + j."""
    rep = q.shape[1] // k.shape[1]
    kk = k.float().repeat_interleave(rep, dim=1)
    vv = v.float().repeat_interleave(rep, dim=1)
    q_len, skv = q.shape[2], k.shape[2]
    logits = (q.float() @ kk.transpose(-1, -2)) * scale                          # [B, H, q_len, Skv]
    pos = torch.arange(q_len, device=q.device)[:, None] + (skv - q_len)
    logits = logits.masked_fill(torch.arange(skv, device=q.device)[None, :] > pos, float("-inf"))
    return (torch.softmax(logits, dim=-1) @ vv).transpose(1, 2)                  # [B, q_len, H, D]


@pytest.mark.parametrize("B,H,Hkv,Skv,q_len,dtype", [
    (2, 8, 2, 1000, 2, torch.bfloat16),       # a few tokens: the decode kernel per token
    (1, 32, 8, 20000, 16, torch.bfloat16),
    (3, 4, 4, 333, 7, torch.float16),
    (2, 6, 2, 1000, 5, torch.bfloat16),       # three query heads per key/value head: the causal tiles
    (2, 8, 2, 1000, 17, torch.bfloat16),      # more tokens: the forward kernel's causal tiles on the tail
    (1, 8, 8, 5000, 300, torch.float16),
    (2, 16, 4, 4097, 1025, torch.bfloat16),
    (1, 4, 2, 700, 699, torch.bfloat16),
    (1, 32, 8, 40000, 4096, torch.bfloat16),  # enough tiles for the resident-workgroup kernel
])
def test_several_new_tokens_against_the_cache(B, H, Hkv, Skv, q_len, dtype):
    from moba_amd.decode import chunk_decode_attention
    print("tail case", B, H, Hkv, Skv, q_len, dtype, flush=True)
    g = torch.Generator(device="cuda").manual_seed(Skv + q_len)
    q = torch.randn((B, H, q_len, 128), generator=g, device="cuda").to(dtype)
    cache_k = torch.randn((B, Hkv, Skv + 50, 128), generator=g, device="cuda").to(dtype)
    cache_v = torch.randn((B, Hkv, Skv + 50, 128), generator=g, device="cuda").to(dtype)
    k, v = cache_k[:, :, :Skv], cache_v[:, :, :Skv]       # a preallocated cache sliced to its filled length
    for scale in (None, 0.15):
        out = chunk_decode_attention(q, k, v, scale)
        want = _ref_tail(q, k, v, 128 ** -0.5 if scale is None else scale)
        assert out.shape == (B, q_len, H, 128) and torch.isfinite(out.float()).all()
        err = (out.float() - want).abs()
        assert err.max() < 2e-2 and err.mean() < 1e-3, (err.max().item(), err.mean().item())


def test_adapter_decodes_several_tokens_with_the_kernels():
    from moba_amd import MoBAConfig, moba_attn_varlen
    from moba_amd.moba_naive import moba_attn_varlen_naive
    from moba_amd.wrapper import moba_layer
    import moba_amd.decode as D

    class Mod(torch.nn.Module):
        is_causal = True

    g = torch.Generator(device="cuda").manual_seed(4)
    cfg = MoBAConfig(64, 3)
    for q_len in (3, 40):
        q = torch.randn((2, 8, q_len, 128), generator=g, device="cuda").to(torch.bfloat16)
        k = torch.randn((2, 2, 333, 128), generator=g, device="cuda").to(torch.bfloat16)
        v = torch.randn((2, 2, 333, 128), generator=g, device="cuda").to(torch.bfloat16)
        calls, real = [], D.chunk_decode_attention
        D.chunk_decode_attention = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
        try:
            a, _ = moba_layer(moba_attn_varlen, cfg, Mod(), q, k, v, None)          # HIP kernels
        finally:
            D.chunk_decode_attention = real
        b, _ = moba_layer(moba_attn_varlen_naive, cfg, Mod(), q, k, v, None)    # SDPA with the bottom-right mask
        assert calls == [1] and a.shape == b.shape == (2, q_len, 8, 128)
        assert (a.float() - b.float()).abs().max() < 2e-2
