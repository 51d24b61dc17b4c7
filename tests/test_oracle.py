"""Pins the CPU oracle (oracle/moba_oracle.py) against what the mathematics and
torch library routines fix.  The reference holds no golden vectors for this path
(its only test is relational: tests/test_moba_attn.py:37-100), so each oracle
function is pinned by closed forms, brute force, library routines and special
cases chosen so that a dropped term / wrong index / transposed operand fails."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

from oracle import moba_oracle as O
from conftest import make_case


# ---------------------------------------------------------------- calc_chunks
@pytest.mark.parametrize("cu,B,cu_chunk,filtered,c2b", [
    ([0, 5, 8], 2, [0, 2, 4, 5, 7, 8], [0, 1, 3], [0, 0, 0, 1, 1]),
    ([0, 4, 8], 2, [0, 2, 4, 6, 8], [0, 2], [0, 0, 1, 1]),
    ([0, 1, 2, 8], 4, [0, 1, 2, 6, 8], [2], [0, 1, 2, 2]),
    ([0, 7], 16, [0, 7], [], [0]),
])
def test_calc_chunks_worked_examples(cu, B, cu_chunk, filtered, c2b):
    m = O.calc_chunks(cu, B)
    assert m["cu_chunk"].tolist() == cu_chunk
    assert m["filtered_chunk_indices"].tolist() == filtered
    assert m["num_filtered_chunk"] == len(filtered)
    assert m["chunk_to_batch"].tolist() == c2b


def test_calc_chunks_invariants_random():
    rng = np.random.default_rng(0)
    for _ in range(200):
        nseq = int(rng.integers(1, 6))
        lens = rng.integers(1, 40, size=nseq)
        B = int(rng.integers(1, 12))
        cu = np.concatenate([[0], np.cumsum(lens)])
        m = O.calc_chunks(cu, B)
        cc = m["cu_chunk"]
        d = np.diff(cc)
        assert (d > 0).all() and (d <= B).all() and cc[-1] == cu[-1]
        assert (d[m["filtered_chunk_indices"]] == B).all()
        assert m["num_filtered_chunk"] == int(sum(math.ceil(L / B) - 1 for L in lens))
        # every sequence boundary is a chunk boundary
        assert set(cu.tolist()) <= set(cc.tolist())


# ---------------------------------------------------------------- chunk mean
def test_chunk_mean_exact_on_integers():
    g = torch.Generator().manual_seed(1)
    k = torch.randint(-8, 9, (96, 2, 16), generator=g).to(torch.bfloat16)
    cu = [0, 40, 96]
    B = 8
    kb = O.chunk_mean(k, cu, B)
    m = O.calc_chunks(cu, B)
    assert kb.shape[0] == m["num_filtered_chunk"] == 4 + 6
    for i, cid in enumerate(m["filtered_chunk_indices"]):
        s0 = int(m["cu_chunk"][cid])
        ref = sum(k[s0 + j].float() for j in range(B)) / B      # exact in fp32: small integers / 8
        assert torch.equal(kb[i].float(), ref.to(torch.bfloat16).float())


def test_chunk_mean_vs_torch_mean():
    q, k, v, _, cu, _ = make_case(3, 1024, 2)
    B = 128
    kb = O.chunk_mean(k, cu, B)
    m = O.calc_chunks(cu, B)
    ref = torch.stack([k[int(m["cu_chunk"][c]):int(m["cu_chunk"][c]) + B].float().mean(0).to(torch.bfloat16)
                       for c in m["filtered_chunk_indices"]])
    # fp32-accumulated torch mean can differ from the exact mean by one bf16 ulp, rarely
    diff = (kb.float() - ref.float()).abs()
    ulp = torch.maximum(kb.float().abs(), ref.float().abs()) * 2 ** -7
    assert (diff <= ulp).all()
    assert (diff == 0).float().mean() > 0.995


def test_chunk_mean_rounds_once():
    """A mean just above the tie between two neighbours of the narrow type: 4 + 2^-6 + 2^-38 over 4 tokens is
    1 + 2^-8 + 2^-40.  One rounding gives the upper neighbour; rounding to fp32 first lands on the tie itself
    (1 + 2^-8), which nearest-even then sends down.  Known answers, bf16 and fp16 (tie of 1 and 1 + 2^-10 is
    1 + 2^-11: 4 + 2^-9 + 2^-24, the smallest fp16), plus the mirror image just below a tie and an exact tie."""
    for dtype, step, tiny in ((torch.bfloat16, 2.0 ** -7, 2.0 ** -38), (torch.float16, 2.0 ** -10, 2.0 ** -24)):
        k = torch.zeros((8, 1, 8), dtype=dtype)
        k[0, 0, :] = 4.0
        k[1, 0, 0] = 2 * step; k[2, 0, 0] = tiny            # just above the tie  -> 1 + step
        k[1, 0, 1] = 2 * step; k[2, 0, 1] = -tiny         # just below the tie  -> 1
        k[1, 0, 2] = 2 * step                                      # the tie itself      -> 1 (even)
        k[1, 0, 3] = 6 * step                                      # tie of 1+step, 1+2step -> 1 + 2 step (even)
        kb = O.chunk_mean(k, [0, 8], 4).double()
        assert kb.shape == (1, 1, 8)
        assert kb[0, 0, 0] == 1 + step and kb[0, 0, 1] == 1.0 and kb[0, 0, 2] == 1.0 and kb[0, 0, 3] == 1 + 2 * step
        assert (kb[0, 0, 4:] == 1.0).all()
    # the helper against exact rational arithmetic on random fp64 values near and far from ties
    from fractions import Fraction
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2000, generator=g, dtype=torch.float64)
    x[:500] = (1 + torch.randint(0, 256, (500,), generator=g).double() * 2.0 ** -8) * (1 + (torch.rand(500, generator=g, dtype=torch.float64) - 0.5) * 2.0 ** -30)
    got = O.round_once(x, torch.bfloat16).double()
    for xi, gi in zip(x.tolist(), got.tolist()):
        f = Fraction(xi)
        e = math.floor(math.log2(abs(xi)))
        ulp = Fraction(2) ** (e - 7)
        lo = (f / ulp).__floor__() * ulp
        hi = lo + ulp
        want = lo if (f - lo < hi - f or (f - lo == hi - f and (lo / ulp) % 2 == 0)) else hi
        assert Fraction(gi) == want, (xi, gi, float(want))


# ---------------------------------------------------------------- gate
def test_gate_scores_bruteforce():
    q, k, v, _, cu, _ = make_case(3, 192, 2, head_dim=16, seed=3)
    B = 16
    kb = O.chunk_mean(k, cu, B)
    gate = O.gate_scores(q, kb, cu, B)
    m = O.calc_chunks(cu, B)
    S, H, F = gate.shape
    cuv = np.asarray(cu)
    for s in range(0, S, 7):
        b = int(np.searchsorted(cuv, s, side="right") - 1)
        for f in range(F):
            cid = int(m["filtered_chunk_indices"][f])
            same_seq = int(m["chunk_to_batch"][cid]) == b
            ends_before = int(m["cu_chunk"][cid + 1]) <= s
            for h in range(H):
                if same_seq and ends_before:
                    ref = float((q[s, h].float() * kb[f, h].float()).sum())
                    assert abs(float(gate[s, h, f]) - ref) < 1e-4 * max(1.0, abs(ref))
                else:
                    assert gate[s, h, f] == O.NEG_INF


# ---------------------------------------------------------------- selection
def test_select_topk_vs_torch_topk_and_fullsort():
    q, k, v, _, cu, _ = make_case(4, 512, 4, seed=5)
    B = 32
    kb = O.chunk_mean(k, cu, B)
    gate = O.gate_scores(q, kb, cu, B)
    S, H, F = gate.shape
    for kk in (1, 2, 3, 7):
        sel = O.select_topk(gate, kk)
        _, ti = torch.topk(gate, k=min(kk, F), dim=-1, largest=True, sorted=False)
        tv = torch.gather(gate, -1, ti)
        for s in range(0, S, 5):
            for h in range(H):
                want = {int(i) for i, val in zip(ti[s, h], tv[s, h]) if val != O.NEG_INF}
                got = {int(x) for x in sel[s, h] if x >= 0}
                assert got == want
                # threshold property against a full sort
                valid = [(float(gate[s, h, f]), f) for f in range(F) if gate[s, h, f] != O.NEG_INF]
                assert len(got) == min(kk, len(valid))
                if got and len(valid) > len(got):
                    lo = min(float(gate[s, h, f]) for f in got)
                    hi = max(sc for sc, f in valid if f not in got)
                    assert lo >= hi


def test_select_topk_count_and_causality():
    q, k, v, _, cu, _ = make_case(4, 512, 2, seed=6)
    B = 32
    kb = O.chunk_mean(k, cu, B)
    sel = O.select_topk(O.gate_scores(q, kb, cu, B), 3)
    m = O.calc_chunks(cu, B)
    cuv = np.asarray(cu)
    for s in range(sel.shape[0]):
        b = int(np.searchsorted(cuv, s, side="right") - 1)
        c = (s - cuv[b]) // B
        fb = int(m["first_filtered"][b])
        for h in range(sel.shape[1]):
            got = [int(x) for x in sel[s, h] if x >= 0]
            assert len(got) == min(3, c)
            assert all(fb <= f < fb + c for f in got)
            assert got == sorted(got)


def test_select_topk_tie_rule():
    gate = torch.tensor([[[1.0, 2.0, 2.0, 2.0, O.NEG_INF]]])
    assert O.select_topk(gate, 2)[0, 0].tolist() == [1, 2]
    assert O.select_topk(gate, 1)[0, 0].tolist() == [1]
    gate = torch.tensor([[[O.NEG_INF, O.NEG_INF, O.NEG_INF]]])
    assert O.select_topk(gate, 2)[0, 0].tolist() == [-1, -1]
    gate = torch.tensor([[[0.5, O.NEG_INF, O.NEG_INF]]])
    assert O.select_topk(gate, 2)[0, 0].tolist() == [0, -1]


# ---------------------------------------------------------------- lists
def test_gather_lists_against_mask_nonzero():
    q, k, v, _, cu, _ = make_case(3, 384, 2, seed=7)
    B = 32
    kb = O.chunk_mean(k, cu, B)
    gate = O.gate_scores(q, kb, cu, B)
    sel = O.select_topk(gate, 2)
    S, H, F = gate.shape
    counts, offs, rows, slots = O.gather_lists(sel, F)
    assert counts.sum() == O.expected_pair_count(cu, B, 2, H) == rows.size
    # the reference's ordering: nonzero of the [F, H*S] view (moba_efficient.py:375-377)
    mask = O.selection_mask(sel, F)
    hs = mask.reshape(F, -1).nonzero(as_tuple=True)[-1]
    assert torch.equal(hs % S, torch.from_numpy(rows))
    assert torch.equal(mask.sum(dim=-1).flatten(), torch.from_numpy(counts))
    for p in range(rows.size):
        seg = int(np.searchsorted(offs, p, side="right") - 1)
        assert int(sel[rows[p], seg % H, slots[p]]) == seg // H


# ---------------------------------------------------------------- attention
def sdpa_causal(q, k, v, cu):
    outs = []
    for a, b in zip(cu[:-1], cu[1:]):
        qq, kk, vv = (x[a:b].float().permute(1, 0, 2)[None] for x in (q, k, v))
        outs.append(Fn.scaled_dot_product_attention(qq, kk, vv, is_causal=True)[0].permute(1, 0, 2))
    return torch.cat(outs)


def test_attend_dense_reduces_to_causal_sdpa_when_all_chunks_selected():
    q, k, v, _, cu, mx = make_case(3, 320, 2, head_dim=32, seed=8)
    B = 32
    # topk-1 >= every sequence's chunk count: every past chunk is selected
    out = O.moba_attn_varlen_oracle(q, k, v, cu, mx, B, 64)
    torch.testing.assert_close(out, sdpa_causal(q, k, v, cu), atol=2e-5, rtol=1e-4)
    # chunk >= longest sequence: fallback (moba_efficient.py:313-321)
    out = O.moba_attn_varlen_oracle(q, k, v, cu, mx, 512, 3)
    torch.testing.assert_close(out, sdpa_causal(q, k, v, cu), atol=2e-5, rtol=1e-4)
    # topk = 1 in the efficient path also means full causal attention
    out = O.moba_attn_varlen_oracle(q, k, v, cu, mx, B, 1)
    torch.testing.assert_close(out, sdpa_causal(q, k, v, cu), atol=2e-5, rtol=1e-4)


def test_attend_dense_uniform_v_and_lse():
    q, k, v, _, cu, mx = make_case(2, 256, 2, head_dim=32, seed=9)
    B = 32
    vu = torch.ones_like(v) * 0.5
    out, lse, sel = O.moba_attn_varlen_oracle(q, k, vu, cu, mx, B, 3, return_aux=True)
    torch.testing.assert_close(out, torch.full_like(out, 0.5), atol=1e-5, rtol=0)
    # LSE = logsumexp over the attended set, by explicit enumeration
    bo, bl = O.attend_blocked(q, k, v, cu, B, sel, rows=np.arange(0, 256, 13))
    torch.testing.assert_close(lse[0:256:13], bl, atol=1e-4, rtol=1e-5)
    o2 = O.attend_dense(q, k, v, cu, B, sel)
    torch.testing.assert_close(o2[0:256:13], bo, atol=1e-4, rtol=1e-4)


def test_attend_dense_gradcheck_fp64():
    g = torch.Generator().manual_seed(10)
    q, k, v = (torch.randn((24, 1, 4), generator=g, dtype=torch.float64, requires_grad=True) for _ in range(3))
    cu = [0, 10, 24]
    sel = torch.full((24, 1, 1), -1, dtype=torch.int32)
    sel[8:10, 0, 0] = 0        # seq 0 (chunks of 4): tokens 8,9 pick chunk 0
    sel[18:24, 0, 0] = 2       # seq 1 first filtered id is 2
    fn = lambda a, b, c: O.attend_dense(a, b, c, cu, 4, sel, dtype=torch.float64)
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-5)


def test_merge_partials_equals_union():
    g = torch.Generator().manual_seed(11)
    qv = torch.randn(5, 16, generator=g)
    kk = torch.randn(40, 16, generator=g)
    vv = torch.randn(40, 16, generator=g)
    logits = qv @ kk.t()
    full = torch.softmax(logits, -1) @ vv
    parts = [(0, 7), (7, 8), (8, 30), (30, 40)]
    outs = torch.stack([torch.softmax(logits[:, a:b], -1) @ vv[a:b] for a, b in parts])
    lses = torch.stack([torch.logsumexp(logits[:, a:b], -1) for a, b in parts])
    out, lse = O.merge_partials(outs, lses)
    torch.testing.assert_close(out, full, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(lse, torch.logsumexp(logits, -1), atol=1e-5, rtol=1e-5)
    # an empty part (lse=-inf, garbage output) must not contribute
    outs2 = torch.cat([outs, torch.full_like(outs[:1], float("nan"))])
    lses2 = torch.cat([lses, torch.full_like(lses[:1], O.NEG_INF)])
    out2, _ = O.merge_partials(outs2, lses2)
    torch.testing.assert_close(out2, full, atol=1e-5, rtol=1e-5)


# ---------------------------------------------------------------- naive formulation
@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [
    (1, 512, 2, 64, 3), (4, 512, 1, 32, 2), (3, 700, 2, 100, 4), (1, 256, 2, 512, 3)])
def test_naive_formulation_agrees_with_selection_formulation(batch, seqlen, heads, B, topk):
    """Two different formulations of the attended set (moba_naive.py:58-81 vs
    moba_efficient.py:352-371) must agree; topk >= 2 where both are defined alike."""
    q, k, v, _, cu, mx = make_case(batch, seqlen, heads, head_dim=32, seed=12)
    a = O.moba_attn_varlen_naive(q, k, v, cu, mx, B, topk).float()
    b = O.moba_attn_varlen_oracle(q, k, v, cu, mx, B, topk)
    # naive rounds its output to bf16
    assert (a - b).abs().max() < 2e-2
    assert (a - b).abs().mean() < 1e-3


def test_naive_topk1_is_chunk_local():
    q, k, v, _, cu, mx = make_case(1, 128, 1, head_dim=16, seed=13)
    B = 32
    a = O.moba_attn_varlen_naive(q, k, v, cu, mx, B, 1).float()
    # chunk-local causal attention == causal SDPA with every chunk as its own sequence
    ref = sdpa_causal(q, k, v, [0, 32, 64, 96, 128])
    assert (a - ref).abs().max() < 2e-2


def test_flop_count_matches_published_closed_forms():
    # figures stated for the benchmark configurations
    assert O.attention_flops([0, 131072], 4096, 12, 32, 128) == pytest.approx(8.301e13, rel=1e-3)
    assert O.attention_flops([0, 32768], 2048, 3, 1, 128) == pytest.approx(7.95e10, rel=1e-2)
    assert O.expected_pair_count([0, 131072], 4096, 11, 32) == 37486592
