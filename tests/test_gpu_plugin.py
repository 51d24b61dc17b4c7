"""The transformers plugin on the GPU: "moba" (HIP kernels) against "moba_naive"
(dense torch ops) on a tiny random-weight Llama built from a local config -- the offline
counterpart of examples/llama.py."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _model(dtype, head_dim=128):
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(vocab_size=128, hidden_size=4 * head_dim, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=2, head_dim=head_dim, max_position_embeddings=2048)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg).to(dtype).cuda().eval()


def test_prefill_logits_full_selection_equals_eager():
    """With topk >= the number of chunks every past chunk is selected, so "moba" must
    reproduce ordinary causal attention through the whole model."""
    from moba_amd import MoBAConfig, register_moba
    register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=16))
    model = _model(torch.bfloat16)
    ids = torch.randint(0, 128, (2, 1024), device="cuda")
    with torch.no_grad():
        model.config._attn_implementation = "eager"
        ref = model(ids).logits.float()
        model.config._attn_implementation = "moba"
        got = model(ids).logits.float()
    err = (got - ref).abs()
    assert err.max() < 6e-2 and err.mean() < 4e-3, (err.max().item(), err.mean().item())


def test_prefill_logits_moba_vs_naive():
    from moba_amd import MoBAConfig, register_moba
    register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=3))
    model = _model(torch.bfloat16)
    ids = torch.randint(0, 128, (2, 1024), device="cuda")
    with torch.no_grad():
        model.config._attn_implementation = "moba_naive"
        ref = model(ids).logits.float()
        model.config._attn_implementation = "moba"
        got = model(ids).logits.float()
    err = (got - ref).abs()
    # Two bf16 pipelines through two layers.  In a random-weight model with a 128-token
    # vocabulary the chunk means are nearly identical, so gate scores are near-ties and a
    # one-ulp difference of a chunk mean flips the selected block for some tokens: bound
    # the typical error tightly and the fraction of flipped tokens loosely.
    assert err.median() < 4e-3 and err.mean() < 8e-3, (err.median().item(), err.mean().item())
    assert (err > 0.1).float().mean() < 2e-2


def test_moba_layer_direct_equals_operator():
    from moba_amd import MoBAConfig, moba_attn_varlen
    from moba_amd.wrapper import moba_layer

    class Mod(torch.nn.Module):
        is_causal = True

    b, hq, hkv, s, d = 2, 4, 2, 512, 128
    g = torch.Generator().manual_seed(1)
    query = torch.randn((b, hq, s, d), generator=g).to(torch.bfloat16).cuda()
    key = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16).cuda()
    value = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16).cuda()
    out, w = moba_layer(moba_attn_varlen, MoBAConfig(64, 3), Mod(), query, key, value, None)
    qf = query.permute(0, 2, 1, 3).reshape(b * s, hq, d)
    kf = key.permute(0, 2, 1, 3).reshape(b * s, hkv, d).repeat_interleave(2, dim=1)
    vf = value.permute(0, 2, 1, 3).reshape(b * s, hkv, d).repeat_interleave(2, dim=1)
    cu = torch.tensor([0, s, 2 * s], dtype=torch.int32, device="cuda")
    ref = moba_attn_varlen(qf, kf, vf, cu, s, 64, 3)
    assert w is None and torch.equal(out, ref)


def test_generate_runs_prefill_then_decode():
    from moba_amd import MoBAConfig, register_moba
    register_moba(MoBAConfig(moba_chunk_size=64, moba_topk=3))
    model = _model(torch.bfloat16)
    model.config._attn_implementation = "moba"
    ids = torch.randint(0, 128, (1, 300), device="cuda")
    import moba_amd.decode as D
    calls, real = [], D.decode_attention

    def counting(query, key, value, scaling=None):
        calls.append(key.shape[2])
        return real(query, key, value, scaling)

    D.decode_attention = counting
    try:
        with torch.no_grad():
            out = model.generate(ids, max_new_tokens=4, do_sample=False)
    finally:
        D.decode_attention = real
    assert out.shape == (1, 304)
    # every decode step of every layer went through the HIP decode kernel, over a growing cache
    assert len(calls) == 3 * model.config.num_hidden_layers and calls[0] == 301 and calls[-1] == 303


def test_narrow_head_model_prefill_and_generate():
    """A model with head_dim 64: the prefill runs the HIP operator on zero-padded heads (full selection, so it
    must reproduce eager attention), decoding goes through PyTorch SDPA (the decode kernel is built for 128)."""
    from moba_amd import MoBAConfig, register_moba
    register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=16))
    model = _model(torch.bfloat16, head_dim=64)
    ids = torch.randint(0, 128, (2, 1024), device="cuda")
    with torch.no_grad():
        model.config._attn_implementation = "eager"
        ref = model(ids).logits.float()
        model.config._attn_implementation = "moba"
        got = model(ids).logits.float()
        out = model.generate(ids[:1, :300], max_new_tokens=3, do_sample=False)
    err = (got - ref).abs()
    assert err.max() < 6e-2 and err.mean() < 4e-3, (err.max().item(), err.mean().item())
    assert out.shape == (1, 303)


def test_full_attention_layers_through_the_hip_operator():
    """Layer-wise hybrid: layers named in full_attention_layers run the HIP operator with one chunk per
    sequence (plain causal attention), the others keep MoBA.  With both layers full the model must reproduce
    eager attention; with one of them full it must agree with the dense "moba_naive" plugin under the same
    configuration, and differ from the all-MoBA run (the switch really changes a layer)."""
    from moba_amd import MoBAConfig, register_moba
    model = _model(torch.bfloat16)
    ids = torch.randint(0, 128, (2, 1024), device="cuda")
    import moba_amd.moba_efficient as E
    chunk_sizes, real = [], E.moba_attn_varlen.batched_impl

    def spying(query, key, value, moba_chunk_size, moba_topk):   # (a batch of two: the adapter's batched path)
        chunk_sizes.append(moba_chunk_size)
        return real(query, key, value, moba_chunk_size, moba_topk)

    E.moba_attn_varlen.batched_impl = spying
    try:
        with torch.no_grad():
            model.config._attn_implementation = "eager"
            eager = model(ids).logits.float()
            register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=3, full_attention_layers=(0, 1)))
            model.config._attn_implementation = "moba"
            both_full = model(ids).logits.float()
            assert chunk_sizes == [1024, 1024]
            register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=3, full_attention_layers=(-1,)))
            del chunk_sizes[:]
            last_full = model(ids).logits.float()
            assert chunk_sizes == [128, 1024]
            model.config._attn_implementation = "moba_naive"
            last_full_naive = model(ids).logits.float()
            register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=3))
            model.config._attn_implementation = "moba"
            none_full = model(ids).logits.float()
    finally:
        E.moba_attn_varlen.batched_impl = real
        register_moba(MoBAConfig(moba_chunk_size=128, moba_topk=3))
    err = (both_full - eager).abs()
    assert err.max() < 6e-2 and err.mean() < 4e-3, (err.max().item(), err.mean().item())
    err = (last_full - last_full_naive).abs()
    assert err.median() < 4e-3 and err.mean() < 8e-3, (err.median().item(), err.mean().item())
    assert (last_full - none_full).abs().max() > 1e-2
