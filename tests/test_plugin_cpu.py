"""Plugin surface and the torch-op "moba_naive" implementation (CPU)."""

import functools

import pytest
import torch

from conftest import make_case
from oracle import moba_oracle as O


def test_package_surface():
    import moba_amd
    from moba_amd import MoBAConfig, moba_attn_varlen, moba_layer, register_moba
    from moba_amd.moba_efficient import moba_attn_varlen as f2
    from moba_amd.moba_naive import moba_attn_varlen_naive
    from moba_amd.wrapper import hf_to_fa, fa_to_hf

    assert moba_attn_varlen is f2
    cfg = MoBAConfig(moba_chunk_size=64, moba_topk=3)
    assert (cfg.moba_chunk_size, cfg.moba_topk) == (64, 3)
    import inspect
    names = list(inspect.signature(moba_attn_varlen).parameters)
    assert names == ["q", "k", "v", "cu_seqlens", "max_seqlen", "moba_chunk_size", "moba_topk"]
    assert list(inspect.signature(moba_attn_varlen_naive).parameters) == names


def test_register_moba_writes_both_keys():
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    from moba_amd import MoBAConfig, register_moba

    register_moba(MoBAConfig(32, 3))
    for key in ("moba", "moba_naive"):
        fn = ALL_ATTENTION_FUNCTIONS[key]
        assert isinstance(fn, functools.partial) and fn.args[1].moba_chunk_size == 32
        assert key in ALL_ATTENTION_FUNCTIONS.valid_keys()


def test_layout_helpers_roundtrip():
    from moba_amd.wrapper import fa_to_hf, hf_to_fa
    x = torch.randn(3, 4, 5, 8)
    y = hf_to_fa(x)
    assert y.shape == (15, 4, 8)
    assert torch.equal(y[5 * 1 + 2, 3], x[1, 3, 2])
    assert torch.equal(fa_to_hf(y, 3), x)


@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [(1, 256, 2, 32, 3), (3, 300, 2, 50, 2), (2, 200, 1, 64, 4)])
def test_naive_impl_matches_oracle(batch, seqlen, heads, B, topk):
    from moba_amd.moba_naive import moba_attn_varlen_naive
    q, k, v, do, cu, mx = make_case(batch, seqlen, heads, head_dim=32, seed=2)
    a = moba_attn_varlen_naive(q, k, v, torch.tensor(cu), mx, B, topk).float()
    b = O.moba_attn_varlen_naive(q, k, v, cu, mx, B, topk).float()
    assert (a - b).abs().max() < 2e-2 and (a - b).abs().mean() < 4e-4


def test_moba_layer_prefill_calls_impl_with_reference_arguments():
    """moba_layer hands the operator packed [B*S, Hq, D] tensors with KV heads repeated
    like HF repeat_kv and cu_seqlens in multiples of the sequence length
    (moba/wrapper.py:54-75)."""
    from moba_amd import MoBAConfig
    from moba_amd.wrapper import moba_layer

    seen = {}

    def impl(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
        seen.update(q=q, k=k, v=v, cu=cu_seqlens, mx=max_seqlen, B=moba_chunk_size, T=moba_topk)
        return q

    class Mod(torch.nn.Module):
        is_causal = True

    b, hq, hkv, s, d = 2, 4, 2, 6, 8
    query, key, value = torch.randn(b, hq, s, d), torch.randn(b, hkv, s, d), torch.randn(b, hkv, s, d)
    out, w = moba_layer(impl, MoBAConfig(4, 3), Mod(), query, key, value, None, dropout=0.0, scaling=None)
    assert w is None and out.shape == (b * s, hq, d)
    assert seen["cu"].tolist() == [0, 6, 12] and seen["cu"].dtype == torch.int32
    assert (seen["mx"], seen["B"], seen["T"]) == (6, 4, 3)
    assert torch.equal(seen["q"][1 * s + 2, 3], query[1, 3, 2])
    # head hq uses kv head hq // rep
    assert torch.equal(seen["k"][0 * s + 5, 3], key[0, 1, 5]) and torch.equal(seen["v"][1 * s + 0, 0], value[1, 0, 0])
    assert out.reshape(b, s, -1).shape == (b, s, hq * d)


def test_moba_layer_hands_grouped_heads_to_an_impl_that_takes_them():
    """An implementation that advertises a grouped-query variant receives k, v with their own
    head count (no repeat_interleave copies); the result layout is unchanged."""
    from moba_amd import MoBAConfig, moba_attn_varlen, moba_attn_varlen_gqa
    from moba_amd.wrapper import moba_layer

    assert moba_attn_varlen.grouped_query_impl is moba_attn_varlen_gqa
    seen = {}

    def impl(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
        raise AssertionError("the grouped variant must be called")

    def grouped(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
        seen.update(k=k, v=v)
        return q

    impl.grouped_query_impl = grouped

    class Mod(torch.nn.Module):
        is_causal = True

    b, hq, hkv, s, d = 2, 4, 2, 6, 8
    query, key, value = torch.randn(b, hq, s, d), torch.randn(b, hkv, s, d), torch.randn(b, hkv, s, d)
    out, _ = moba_layer(impl, MoBAConfig(4, 3), Mod(), query, key, value, None)
    assert out.shape == (b * s, hq, d)
    assert seen["k"].shape == (b * s, hkv, d) and torch.equal(seen["k"][1 * s + 2, 1], key[1, 1, 2])


def test_moba_layer_prefill_under_inference_mode():
    """Under torch.inference_mode() the adapter still hands the operator an ordinary cu_seqlens tensor (made
    outside the mode), so that the planner remembers it by identity and no layer reads it back from the device;
    an inference tensor from another caller is planned by value (tests/test_plan.py)."""
    from moba_amd import MoBAConfig
    from moba_amd.plan import make_plan
    from moba_amd.wrapper import moba_layer

    seen = {}

    def impl(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
        seen["plan"] = make_plan(cu_seqlens, moba_chunk_size, moba_topk, device="cpu")
        seen["again"] = make_plan(cu_seqlens, moba_chunk_size, moba_topk, device="cpu")
        seen["inference"] = cu_seqlens.is_inference()
        return q

    impl.takes_host_lengths = True

    class Mod(torch.nn.Module):
        is_causal = True

    b, h, s, d = 2, 2, 7, 8     # a shape no other test uses: the adapter makes a fresh cu_seqlens for it
    with torch.inference_mode():
        x = torch.randn(b, h, s, d)
        out, _ = moba_layer(impl, MoBAConfig(4, 3), Mod(), x, x, x, None)
    assert not seen["inference"] and seen["plan"].cu == [0, 7, 14] and out.shape == (b * s, h, d)
    assert seen["again"] is seen["plan"]


def test_full_attention_layers_switch():
    """Layers named in full_attention_layers get one chunk per sequence (= causal attention in every
    implementation); the others keep the configured chunk size.  Negative indices count from the end."""
    from types import SimpleNamespace
    from moba_amd import MoBAConfig
    from moba_amd.moba_naive import moba_attn_varlen_naive
    from moba_amd.wrapper import moba_layer

    cfg = MoBAConfig(4, 2, full_attention_layers=[0, -1])
    assert cfg.is_full_attention_layer(0, 6) and cfg.is_full_attention_layer(5, 6)
    assert not cfg.is_full_attention_layer(3, 6) and not MoBAConfig(4, 2).is_full_attention_layer(0, 6)
    seen = []

    def impl(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk):
        seen.append(moba_chunk_size)
        return moba_attn_varlen_naive(q, k, v, cu_seqlens, max_seqlen, moba_chunk_size, moba_topk)

    class Mod(torch.nn.Module):
        is_causal = True

        def __init__(self, idx):
            super().__init__()
            self.layer_idx = idx
            self.config = SimpleNamespace(num_hidden_layers=6)

    b, h, s, d = 1, 2, 24, 8
    query, key, value = torch.randn(b, h, s, d), torch.randn(b, h, s, d), torch.randn(b, h, s, d)
    full, _ = moba_layer(impl, cfg, Mod(5), query, key, value, None)
    sparse, _ = moba_layer(impl, cfg, Mod(2), query, key, value, None)
    assert seen == [24, 4]
    mask = torch.tril(torch.ones(s, s, dtype=torch.bool))
    ref = torch.softmax((query @ key.transpose(-1, -2) / d ** 0.5).masked_fill(~mask, float("-inf")), -1) @ value
    torch.testing.assert_close(full.view(b, s, h, d).transpose(1, 2), ref, atol=1e-5, rtol=1e-5)
    assert not torch.allclose(sparse.view(b, s, h, d).transpose(1, 2), ref, atol=1e-3)


def test_moba_layer_decode_is_full_attention():
    from moba_amd import MoBAConfig
    from moba_amd.wrapper import moba_layer

    class Mod(torch.nn.Module):
        is_causal = True

    b, hq, hkv, s, d = 1, 4, 2, 9, 16
    query = torch.randn(b, hq, 1, d)
    key, value = torch.randn(b, hkv, s, d), torch.randn(b, hkv, s, d)
    out, _ = moba_layer(None, MoBAConfig(4, 2), Mod(), query, key, value, None, dropout=0.0, scaling=None)
    kk = key.repeat_interleave(2, dim=1)
    vv = value.repeat_interleave(2, dim=1)
    ref = torch.softmax(query @ kk.transpose(-1, -2) / d ** 0.5, -1) @ vv
    assert out.shape == (b, 1, hq, d)
    torch.testing.assert_close(out, ref.transpose(1, 2), atol=1e-5, rtol=1e-5)


def test_tiny_llama_runs_with_moba_naive_plugin():
    """Offline counterpart of examples/llama.py: a random-weight Llama built from a local
    config, attention routed through the registered "moba_naive" plugin; with topk >= the
    chunk count MoBA is exactly causal attention, so logits must match eager attention."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from moba_amd import MoBAConfig, register_moba

    register_moba(MoBAConfig(moba_chunk_size=8, moba_topk=16))
    cfg = LlamaConfig(vocab_size=64, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=128)
    torch.manual_seed(0)
    cfg._attn_implementation = "eager"
    model = LlamaForCausalLM(cfg).eval()
    ids = torch.randint(0, 64, (2, 40))
    with torch.no_grad():
        ref = model(ids).logits
        model.config._attn_implementation = "moba_naive"
        got = model(ids).logits
    torch.testing.assert_close(got, ref, atol=2e-4, rtol=2e-4)
