"""End-to-end parity of moba_attn_varlen (forward + backward) against the CPU oracle,
reproducing the reference's own test matrix and data recipe
(tests/test_moba_attn.py:8-42) and its tolerances (:85-100).  GPU only; every call
goes through the C ABI."""

import itertools
import os

import numpy as np
import pytest
import torch

from conftest import make_case
from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu

# tolerances: max-abs 2e-2 and mean-abs 2e-3 against the fp32 oracle, and the reference test's own bounds
MAX_ABS, MEAN_ABS = 2e-2, 2e-3
REF_MAX_ABS, REF_MEAN_ABS = 4e-2, 4e-4


class dense_prefix:
    """The operator's choice between a batch's plain plan and the one with dense prefixes, for the calls inside:
    True / False force it, None leaves it to the operator (dense prefixes for large problems only)."""

    def __init__(self, choice):
        self.choice = choice

    def __enter__(self):
        from moba_amd import moba_efficient as E
        self.saved = E.DENSE_PREFIX
        E.DENSE_PREFIX = self.choice

    def __exit__(self, *exc):
        from moba_amd import moba_efficient as E
        E.DENSE_PREFIX = self.saved
        return False


def check_selection(sel, want, gate, tol=1e-4):
    """The kernel's selection against the oracle's: equal as sets except where the fp32 scores nearly tie."""
    got = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got = torch.where(got == 1 << 30, torch.full_like(got, -1), got)
    diff_rows = (got != want).any(dim=-1)
    for s_, h_ in diff_rows.nonzero().tolist():
        a = set(got[s_, h_].tolist()) - {-1}
        b = set(want[s_, h_].tolist()) - {-1}
        gap = max(abs(float(gate[s_, h_, x]) - float(gate[s_, h_, y])) for x in a ^ b for y in a ^ b)
        assert gap < tol, (s_, h_, a, b, gap)
    assert diff_rows.float().mean() < 1e-3


def run_case(batch, seqlen, heads, B, topk, seed=0, check_grad=True, dtype=torch.bfloat16, ref_bounds=True, dense=None):
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan

    q, k, v, do, cu, mx = make_case(batch, seqlen, heads, seed=seed, dtype=dtype)
    dev = torch.device("cuda")
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    qg, kg, vg = (x.to(dev).requires_grad_(True) for x in (q, k, v))
    with dense_prefix(dense):
        out = E.moba_attn_varlen(qg, kg, vg, cu_t, mx, moba_chunk_size=B, moba_topk=topk)
        if check_grad:
            torch.autograd.backward(out, do.to(dev))
    plan = make_plan(cu_t, B, topk)
    sel = None
    if not plan.fallback:
        sel = E.gate_topk(qg.detach(), E.chunk_mean(kg.detach(), plan), plan).cpu()
        # the kernel's selection must agree with the oracle's except at numerical near-ties
        gate = O.gate_scores(q, O.chunk_mean(k, cu, B), cu, B)
        check_selection(sel, O.select_topk(gate, plan.K), gate)
    qc, kc, vc = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = O.moba_attn_varlen_oracle(qc, kc, vc, cu, mx, B, topk, sel=sel)
    err = (out.detach().cpu().float() - ref.detach()).abs()
    assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, ("out", err.max().item(), err.mean().item())
    # the reference test compares two bf16 outputs (moba_naive returns o.type_as(q)): round the oracle likewise
    err16 = (out.detach().cpu().float() - ref.detach().to(dtype).float()).abs()
    # (those bounds belong to the reference's grid, where every row averages hundreds of keys)
    if ref_bounds:
        assert err16.max() < REF_MAX_ABS and err16.mean() < REF_MEAN_ABS, ("out16", err16.max().item(), err16.mean().item())
    if check_grad:
        ref.backward(do.float())
        got_g = torch.stack([qg.grad.cpu().float(), kg.grad.cpu().float(), vg.grad.cpu().float()], dim=1)
        ref_g = torch.stack([qc.grad, kc.grad, vc.grad], dim=1)
        gerr = (got_g - ref_g).abs()
        if ref_bounds:
            assert gerr.max() < REF_MAX_ABS and gerr.mean() < REF_MEAN_ABS, ("grad", gerr.max().item(), gerr.mean().item())
        else:
            assert gerr.mean() < MEAN_ABS, ("grad", gerr.mean().item())
        # per-tensor, relative to the tensor's scale
        for i, name in enumerate(("dq", "dk", "dv")):
            e = gerr[:, i]
            scale = ref_g[:, i].abs().max().clamp_min(1.0)
            assert e.max() < MAX_ABS * scale, (name, e.max().item(), scale.item())
    return err


GRID = list(itertools.product([1, 4, 7], [1, 2, 4, 8], [512, 1024, 2048], [128, 256, 1024], [2, 3, 4]))


@pytest.mark.parametrize("dense", [None, True])
@pytest.mark.parametrize("chunk", range(12))
def test_reference_grid(chunk, dense):
    """The reference's 324 cases (batch x heads x seqlen x chunk x topk), 27 per test; as the operator plans them
    (problems this small: the reference's own decomposition) and with dense prefixes forced."""
    cases = GRID[chunk * 27:(chunk + 1) * 27]
    for batch, heads, seqlen, B, topk in cases:
        print("case", batch, heads, seqlen, B, topk, dense, flush=True)
        run_case(batch, seqlen, heads, B, topk, dense=dense)


@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [
    (3, 1500, 3, 100, 3),      # chunk size that is not a multiple of any tile size
    (1, 2048, 2, 128, 1),      # topk = 1: full causal attention, as the efficient reference path
    (2, 4096, 2, 64, 12),      # many chunks, k = 11
    (5, 2000, 2, 128, 64),     # topk beyond the chunk count: everything selected
    (6, 777, 5, 96, 2),        # odd sizes, 1-token tails
    (1, 8192, 1, 512, 3),
    (1, 4096, 1, 64, 24),      # k = 23: the 32-entry selection lists
    (2, 4096, 2, 32, 40),      # k = 39: the 64-entry selection lists, 64 chunks per sequence
])
def test_edge_shapes(batch, seqlen, heads, B, topk):
    run_case(batch, seqlen, heads, B, topk, seed=7)
    run_case(batch, seqlen, heads, B, topk, seed=7, dense=True)


@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [
    (1, 1024, 2, 128, 3),
    (4, 2048, 4, 256, 4),
    (7, 2048, 8, 128, 2),
    (3, 1500, 3, 100, 3),
    (1, 2048, 2, 128, 1),
    (2, 4096, 2, 64, 12),
])
def test_float16(batch, seqlen, heads, B, topk):
    """fp16 inputs (the dtype of the reference's example script), same bounds as bf16."""
    run_case(batch, seqlen, heads, B, topk, seed=11, dtype=torch.float16)
    run_case(batch, seqlen, heads, B, topk, seed=11, dtype=torch.float16, dense=True)


@pytest.mark.parametrize("batch,seqlen,heads,kv_heads,B,topk,dtype", [
    (1, 1024, 4, 1, 128, 3, torch.bfloat16),
    (3, 2048, 8, 2, 256, 3, torch.bfloat16),
    (2, 1500, 6, 3, 100, 4, torch.bfloat16),
    (4, 2048, 8, 2, 128, 2, torch.float16),
    (1, 2048, 4, 2, 128, 1, torch.bfloat16),     # fallback: full causal attention
    (2, 65536, 8, 2, 1024, 4, torch.float16),    # enough tiles for the resident-workgroup kernels, fp16
    (1, 8192, 2, 1, 1024, 3, torch.float16),     # few tiles: the forward cuts the history tiles' keys into parts
])
def test_grouped_query(batch, seqlen, heads, kv_heads, B, topk, dtype):
    """k, v with fewer heads: same result (bit for bit in the forward) as expanding them with
    repeat_interleave first (moba/wrapper.py:59-61); dk, dv equal the sums over each group within rounding."""
    from moba_amd import moba_attn_varlen, moba_attn_varlen_gqa
    rep = heads // kv_heads
    q, _, _, do, cu, mx = make_case(batch, seqlen, heads, seed=5, dtype=dtype)
    _, k, v, _, _, _ = make_case(batch, seqlen, kv_heads, seed=6, dtype=dtype)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qa, ka, va = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out_a = moba_attn_varlen_gqa(qa, ka, va, cu_t, mx, B, topk)
    out_a.backward(do.cuda())
    qb = q.cuda().requires_grad_(True)
    kb = torch.repeat_interleave(k.cuda(), rep, dim=1).requires_grad_(True)
    vb = torch.repeat_interleave(v.cuda(), rep, dim=1).requires_grad_(True)
    out_b = moba_attn_varlen(qb, kb, vb, cu_t, mx, B, topk)
    out_b.backward(do.cuda())
    assert torch.equal(out_a, out_b)
    assert torch.equal(qa.grad, qb.grad)
    for ga, gb in ((ka.grad, kb.grad), (va.grad, vb.grad)):
        want = gb.float().view(seqlen, kv_heads, rep, 128).sum(2)
        err = (ga.float() - want).abs()
        assert err.max() <= 2e-2 * want.abs().max().clamp_min(1.0), err.max().item()
        assert err.mean() <= 4e-3 * want.abs().mean() + 1e-6, (err.mean().item(), want.abs().mean().item())
    with pytest.raises(ValueError):
        moba_attn_varlen(qa, ka, va, cu_t, mx, B, topk)       # the 7-argument operator keeps the reference's contract


@pytest.mark.parametrize("batch,seqlen,heads,kv_heads,B,topk,dtype", [
    (1, 1024, 4, 1, 128, 3, torch.bfloat16),
    (3, 2048, 8, 2, 256, 3, torch.bfloat16),
    (2, 1500, 6, 3, 100, 4, torch.float16),
    (4, 2048, 8, 2, 128, 2, torch.float16),
    (1, 2048, 4, 2, 128, 1, torch.bfloat16),     # fallback: full causal attention
    (1, 8192, 2, 1, 1024, 3, torch.bfloat16),    # few tiles: the forward cuts the history tiles' keys into parts
])
@pytest.mark.parametrize("dense", [None, True])
def test_grouped_query_vs_oracle(batch, seqlen, heads, kv_heads, B, topk, dtype, dense):
    """The grouped-query operator against the oracle run on key/value heads expanded with repeat_interleave
    (the reference's semantics, moba/wrapper.py:59-61): out and dq as they are, dk and dv against the
    oracle's gradients summed over the query heads of each group."""
    from moba_amd import moba_attn_varlen_gqa
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    rep = heads // kv_heads
    q, _, _, do, cu, mx = make_case(batch, seqlen, heads, seed=5, dtype=dtype)
    _, k, v, _, _, _ = make_case(batch, seqlen, kv_heads, seed=6, dtype=dtype)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    with dense_prefix(dense):
        out = moba_attn_varlen_gqa(qg, kg, vg, cu_t, mx, B, topk)
        out.backward(do.cuda())
    plan = make_plan(cu_t, B, topk)
    sel = None
    if not plan.fallback:
        sel = E.gate_topk(qg.detach(), E.chunk_mean(kg.detach(), plan), plan).cpu()
        # the selection itself: the oracle's on the expanded heads, up to near-ties of the fp32 scores
        kx = torch.repeat_interleave(k, rep, dim=1)
        gate = O.gate_scores(q, O.chunk_mean(kx, cu, B), cu, B)
        check_selection(sel, O.select_topk(gate, plan.K), gate)
    qc = q.clone().requires_grad_(True)
    kc, vc = (x.clone().requires_grad_(True) for x in (k, v))
    ref = O.moba_attn_varlen_oracle(qc, torch.repeat_interleave(kc, rep, dim=1), torch.repeat_interleave(vc, rep, dim=1),
                                    cu, mx, B, topk, sel=sel)
    ref.backward(do.float())       # autograd of repeat_interleave sums each group's gradients into kc, vc
    err = (out.detach().cpu().float() - ref.detach()).abs()
    assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, ("out", err.max().item(), err.mean().item())
    for name, got_g, want_g in (("dq", qg.grad, qc.grad), ("dk", kg.grad, kc.grad), ("dv", vg.grad, vc.grad)):
        assert got_g.shape == want_g.shape
        e = (got_g.cpu().float() - want_g.float()).abs()
        scale = want_g.abs().max().clamp_min(1.0)
        assert e.max() < MAX_ABS * scale and e.mean() < MEAN_ABS * rep, (name, e.max().item(), e.mean().item(), scale.item())


def test_baseline_config_1():
    """One sequence of 4096 tokens, 4 heads, chunk 512, top-k 3, bf16 N(0,1) from a seed: forward against
    the dense oracle (the configuration the reference's naive path runs on a CPU)."""
    run_case(1, 4096, 4, 512, 3, seed=0, check_grad=False)


def test_baseline_config_2():
    """The reference's own speed-test shape (tests/test_moba_speedup.py:84, README.md:62): one sequence of
    32768 tokens, 1 head, chunk 2048, top-k 3; forward and backward with dO ~ N(0,1) against the dense oracle."""
    run_case(1, 32768, 1, 2048, 3, seed=0, check_grad=True)


@pytest.mark.parametrize("seed", range(4))
def test_random_shapes(seed):
    """Seeded random shapes: odd sequence lengths, chunk sizes that divide nothing, one to many
    sequences, both dtypes; forward and backward against the oracle."""
    rng = np.random.default_rng(100 + seed)
    for _ in range(8):
        seqlen = int(rng.integers(40, 3000))
        batch = int(rng.integers(1, min(9, seqlen // 4)))
        heads = int(rng.integers(1, 6))
        B = int(rng.integers(8, 300))
        topk = int(rng.integers(1, 9))
        dtype = torch.float16 if rng.integers(0, 2) else torch.bfloat16
        dense = bool(rng.integers(0, 2))
        print("random case", batch, seqlen, heads, B, topk, dtype, dense, flush=True)
        run_case(batch, seqlen, heads, B, topk, seed=int(rng.integers(0, 1000)), dtype=dtype, ref_bounds=False, dense=dense)


def test_peaked_softmax_and_exact_gate_ties():
    """(a) Scores with a large spread (q, k scaled by 6: near one-hot softmax, running max far from
    the first tile's) stay within the tolerances.  (b) Keys that repeat with the chunk period give
    every chunk the same representative, hence exactly tied gate scores: the tie rule (lower chunk
    id) must then pick the same chunks as the oracle, bit for bit."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    q, k, v, do, cu, mx = make_case(2, 2048, 2, seed=21)
    q, k = (q.float() * 6).to(torch.bfloat16), (k.float() * 6).to(torch.bfloat16)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    B, topk = 128, 4
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = E.moba_attn_varlen(qg, kg, vg, cu_t, mx, B, topk)
    out.backward(do.cuda())
    plan = make_plan(cu_t, B, topk)
    sel = E.gate_topk(qg.detach(), E.chunk_mean(kg.detach(), plan), plan).cpu()
    qc, kc, vc = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = O.moba_attn_varlen_oracle(qc, kc, vc, cu, mx, B, topk, sel=sel)
    ref.backward(do.float())
    assert torch.isfinite(out.float()).all() and torch.isfinite(qg.grad.float()).all()
    err = (out.detach().cpu().float() - ref.detach().float()).abs()
    assert err.max() < 3e-2 and err.mean() < MEAN_ABS, (err.max().item(), err.mean().item())
    for a, b in ((qg.grad, qc.grad), (kg.grad, kc.grad), (vg.grad, vc.grad)):
        e = (a.cpu().float() - b.float()).abs()
        assert e.max() < 3e-2 * b.float().abs().max().clamp_min(1.0) and e.mean() < 2e-2 * b.float().abs().mean() + 1e-4

    # (b) exact ties
    S, H, B = 1024, 2, 64
    g = torch.Generator().manual_seed(5)
    blk = torch.randn((B, H, 128), generator=g).to(torch.bfloat16)
    k = blk.repeat(S // B, 1, 1)
    q = torch.randn((S, H, 128), generator=g).to(torch.bfloat16)
    cu = [0, S]
    plan = make_plan(cu, B, 4, device="cuda")
    sel = E.gate_topk(q.cuda(), E.chunk_mean(k.cuda(), plan), plan).cpu()
    got = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got = torch.where(got == 1 << 30, torch.full_like(got, -1), got)
    want = O.select_topk(O.gate_scores(q, O.chunk_mean(k, cu, B), cu, B), plan.K)
    assert torch.equal(got, want.to(got.dtype))
    tok = torch.arange(S)
    c = tok // B
    for j in range(plan.K):                       # lowest ids win: slot j holds chunk j wherever it exists
        assert torch.equal(got[:, :, j], torch.where(c > j, torch.tensor(j), torch.tensor(-1))[:, None].expand(S, H).to(got.dtype))


def test_one_token_sequences():
    from moba_amd import moba_efficient as E
    g = torch.Generator().manual_seed(3)
    S, H = 300, 2
    q, k, v = (torch.randn((S, H, 128), generator=g).to(torch.bfloat16) for _ in range(3))
    cu = [0, 1, 2, 130, 131, 300]
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    out = E.moba_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu_t, 169, 32, 3).cpu().float()
    # a 1-token sequence attends only itself
    assert torch.equal(out[0], v[0].float()) and torch.equal(out[130], v[130].float())
    ref = O.moba_attn_varlen_oracle(q, k, v, cu, 169, 32, 3)
    assert (out - ref).abs().max() < MAX_ABS


def test_uniform_v_gives_v():
    from moba_amd import moba_efficient as E
    q, k, v, do, cu, mx = make_case(3, 2048, 2, seed=11)
    v = torch.full_like(v, 0.75)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    out = E.moba_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu_t, mx, 128, 3).cpu().float()
    assert (out - 0.75).abs().max() < 4e-3


def test_backward_is_deterministic():
    from moba_amd import moba_efficient as E
    q, k, v, do, cu, mx = make_case(4, 4096, 4, seed=13)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    grads = []
    for _ in range(2):
        qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
        out = E.moba_attn_varlen(qg, kg, vg, cu_t, mx, 256, 4)
        out.backward(do.cuda())
        grads.append([out.detach().clone(), qg.grad.clone(), kg.grad.clone(), vg.grad.clone()])
    for a, b in zip(*grads):
        assert torch.equal(a, b)


def test_history_tiles_of_dq_cut_into_parts():
    """With few tiles per workgroup the dQ kernel cuts the keys of every history tile into parts that are tiles of
    their own, each leaving its partial dQ in slot rows of its own: 1, 2 and 4 parts give the same out, dk and dv
    bit for bit and a dq that differs by the rounding of the parts' partial sums only; dq lies within the tolerance
    of the oracle for each.  Three sequences with partial last chunks, grouped-query heads."""
    from moba_amd import _lib, moba_attn_varlen_gqa
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    heads, kv_heads, B, topk = 2, 1, 1024, 3
    q, _, _, do, cu, mx = make_case(3, 16384, heads, seed=23)
    _, k, v, _, _, _ = make_case(3, 16384, kv_heads, seed=24)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    lib = _lib.load()
    plan = make_plan(cu_t, B, topk)
    proposed = lib.moba_bwd_dq_key_split(16384, heads, plan.K, B, plan.hist_tile_bound(heads), plan.self_tiles)
    assert proposed in (1, 2, 4, 8) and (proposed == 2 or "MOBA_RESIDENT_CUS" in os.environ)

    def run(split):
        real = lib.moba_bwd_dq_key_split
        plan.memo.clear()   # (the operator keeps the split with the plan)
        try:
            lib.moba_bwd_dq_key_split = lambda *a: split
            qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
            out = moba_attn_varlen_gqa(qg, kg, vg, cu_t, mx, B, topk)
            out.backward(do.cuda())
        finally:
            lib.moba_bwd_dq_key_split = real
            plan.memo.clear()
        return out.detach(), qg.grad, kg.grad, vg.grad

    whole, two, four = run(1), run(2), run(4)
    for cut in (two, four):
        assert torch.equal(cut[0], whole[0]) and torch.equal(cut[2], whole[2]) and torch.equal(cut[3], whole[3])
        e = (cut[1].float() - whole[1].float()).abs()
        assert 0 < e.max() <= 2.0 ** -6 * whole[1].float().abs().max(), e.max().item()
    again = run(2)
    assert torch.equal(again[1], two[1])
    with pytest.raises(RuntimeError, match="moba_bwd"):
        run(3)           # not a power of two
    with pytest.raises(RuntimeError, match="moba_bwd"):
        run(32)          # B is not a multiple of 64 * 32 (and 8 is the most)
    sel = E.gate_topk(q.cuda(), E.chunk_mean(k.cuda(), plan), plan).cpu()
    qc = q.clone().requires_grad_(True)
    rep = heads // kv_heads
    ref = O.moba_attn_varlen_oracle(qc, torch.repeat_interleave(k, rep, dim=1), torch.repeat_interleave(v, rep, dim=1),
                                    cu, mx, B, topk, sel=sel)
    ref.backward(do.float())
    for got in (whole, two, four):
        e = (got[1].cpu().float() - qc.grad.float()).abs()
        scale = qc.grad.abs().max().clamp_min(1.0)
        assert e.max() < MAX_ABS * scale and e.mean() < MEAN_ABS, (e.max().item(), e.mean().item())


def test_key_tiles_cut_into_parts():
    """With few key tiles (here 16384 tokens x 1 key/value head = 128 tiles on 256 compute units) the dK/dV kernel
    cuts every tile into parts that leave fp32 sums for a reduction kernel: grouped-query heads, three sequences
    with partial last chunks.  The result is deterministic, equals the uncut kernel's up to the rounding of the
    different summation order, and both lie within the tolerance of the oracle."""
    from moba_amd import _lib, moba_attn_varlen_gqa
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    heads, kv_heads, B, topk = 2, 1, 1024, 3
    q, _, _, do, cu, mx = make_case(3, 16384, heads, seed=21)
    _, k, v, _, _, _ = make_case(3, 16384, kv_heads, seed=22)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    lib = _lib.load()
    plan = make_plan(cu_t, B, topk)
    if lib.moba_bwd_dkv_scratch_bytes(16384, kv_heads, plan.self_tiles) == 0:
        assert "MOBA_RESIDENT_CUS" in os.environ     # (only the diagnostic that shrinks the chip turns the parts off)
        pytest.skip("the key tiles are not cut with MOBA_RESIDENT_CUS set")

    def run():
        qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
        out = moba_attn_varlen_gqa(qg, kg, vg, cu_t, mx, B, topk)
        out.backward(do.cuda())
        return out.detach(), qg.grad, kg.grad, vg.grad

    cut, again = run(), run()
    for a, b in zip(cut, again):
        assert torch.equal(a, b)
    real = lib.moba_bwd_dkv_scratch_bytes
    try:
        lib.moba_bwd_dkv_scratch_bytes = lambda *a: 0   # no scratch: every key tile in one piece
        whole = run()
    finally:
        lib.moba_bwd_dkv_scratch_bytes = real
    assert torch.equal(cut[0], whole[0]) and torch.equal(cut[1], whole[1])
    for name, a, b in (("dk", cut[2], whole[2]), ("dv", cut[3], whole[3])):
        e = (a.float() - b.float()).abs()
        assert e.max() <= 2.0 ** -7 * b.float().abs().max() and (e > 0).float().mean() < 0.05, (name, e.max().item())
    # ... and the oracle, on expanded key/value heads with the kernel's own selection
    sel = E.gate_topk(q.cuda(), E.chunk_mean(k.cuda(), plan), plan).cpu()
    qc = q.clone().requires_grad_(True)
    kc, vc = (x.clone().requires_grad_(True) for x in (k, v))
    rep = heads // kv_heads
    ref = O.moba_attn_varlen_oracle(qc, torch.repeat_interleave(kc, rep, dim=1), torch.repeat_interleave(vc, rep, dim=1),
                                    cu, mx, B, topk, sel=sel)
    ref.backward(do.float())
    for name, got_g, want_g in (("dk", cut[2], kc.grad), ("dv", cut[3], vc.grad)):
        e = (got_g.cpu().float() - want_g.float()).abs()
        scale = want_g.abs().max().clamp_min(1.0)
        assert e.max() < MAX_ABS * scale and e.mean() < MEAN_ABS * rep, (name, e.max().item(), e.mean().item())


def test_float16_large_gradients_stay_finite():
    """dQ = scale * dS K is summed from per-chunk partials kept in the element type.  The partials are
    scaled before they are rounded, so they leave the fp16 range only where dQ itself would: here
    dQ / scale reaches 2.5e5 (beyond fp16) while dQ stays near 2e4."""
    from moba_amd import moba_efficient as E
    q, k, v, do, cu, mx = make_case(1, 512, 2, seed=5, dtype=torch.float16)
    q = (q.float() * 1e-3).half()
    k = (k.float() * 300).half()
    v = (v.float() * 30).half()
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = E.moba_attn_varlen(qg, kg, vg, cu_t, mx, moba_chunk_size=128, moba_topk=2)
    out.backward(do.cuda())
    qc, kc, vc = (x.float().clone().requires_grad_(True) for x in (q, k, v))
    ref = O.moba_attn_varlen_oracle(qc, kc, vc, cu, mx, 128, 2)
    ref.backward(do.float())
    assert qc.grad.abs().max() * 128 ** 0.5 > 65504 > qc.grad.abs().max()   # the case is what it claims to be
    for got, want in ((out, ref), (qg.grad, qc.grad), (kg.grad, kc.grad), (vg.grad, vc.grad)):
        got = got.detach().cpu().float()
        assert torch.isfinite(got).all()
        assert (got - want.detach()).abs().max() <= 1e-2 * want.detach().abs().max()


@pytest.mark.parametrize("head_dim,dtype", [(64, torch.bfloat16), (96, torch.float16), (40, torch.bfloat16)])
def test_narrow_heads_are_padded(head_dim, dtype):
    """head_dim below 128: zero padding inside the operator, softmax scale head_dim ** -0.5 (the oracle's
    scale for these inputs), outputs and gradients of the narrow shape."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    q, k, v, do, cu, mx = make_case(3, 1500, 4, head_dim=head_dim, seed=21, dtype=dtype)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out = E.moba_attn_varlen(qg, kg, vg, cu_t, mx, moba_chunk_size=128, moba_topk=3)
    assert out.shape == q.shape and out.is_contiguous()
    out.backward(do.cuda())
    # the selection the GPU made on the padded tensors (the gate does not see the zeros)
    plan = make_plan(cu_t, 128, 3)
    pad = (0, 128 - head_dim)
    qp, kp = (torch.nn.functional.pad(x.cuda(), pad) for x in (q, k))
    sel = E.gate_topk(qp, E.chunk_mean(kp, plan), plan).cpu()
    qc, kc, vc = (x.clone().requires_grad_(True) for x in (q, k, v))
    ref = O.moba_attn_varlen_oracle(qc, kc, vc, cu, mx, 128, 3, sel=sel)
    ref.backward(do.float())
    for name, got, want in (("out", out, ref), ("dq", qg.grad, qc.grad), ("dk", kg.grad, kc.grad), ("dv", vg.grad, vc.grad)):
        assert got.shape == want.shape
        err = (got.detach().cpu().float() - want.detach().float()).abs()
        assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, (name, err.max().item(), err.mean().item())
    # and the selection itself is the oracle's on the narrow tensors, up to near-ties of the fp32 scores
    gate = O.gate_scores(q, O.chunk_mean(k, cu, 128), cu, 128)
    check_selection(sel, O.select_topk(gate, plan.K), gate)


def test_heads_wider_than_128_are_refused():
    from moba_amd import moba_attn_varlen
    q, k, v, _, cu, mx = make_case(1, 256, 1, head_dim=192, seed=3)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError, match="head_dim"):
        moba_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu_t, mx, 64, 2)


def test_argument_validation():
    from moba_amd import moba_attn_varlen
    q = torch.zeros((64, 2, 128), dtype=torch.bfloat16, device="cuda")
    cu = torch.tensor([0, 64], dtype=torch.int32, device="cuda")
    with pytest.raises(TypeError):
        moba_attn_varlen(q.float(), q.float(), q.float(), cu, 64, 16, 2)
    with pytest.raises(ValueError):
        moba_attn_varlen(q, q[:, :1], q, cu, 64, 16, 2)
    with pytest.raises(ValueError):
        moba_attn_varlen(q, q, q, torch.tensor([0, 32], dtype=torch.int32, device="cuda"), 64, 16, 2)
    with pytest.raises(RuntimeError):
        moba_attn_varlen(q.cpu(), q.cpu(), q.cpu(), cu, 64, 16, 2)


@pytest.mark.parametrize("layout", ["qkv_slices", "head_major", "gqa_head_major", "mixed", "unaligned"])
def test_strided_inputs(layout):
    """q, k, v that are views with token and head strides (slices of a fused qkv projection, a
    [heads, tokens, dim] cache seen token-first) are read where they lie -- flash-attn does the same
    for the reference (moba/moba_efficient.py:89-128) -- and give bit for bit the result and the
    gradients of packed copies.  Layouts the kernels cannot address are copied, with the same result."""
    from moba_amd import moba_attn_varlen, moba_attn_varlen_gqa
    from moba_amd import moba_efficient as E

    seqlen, heads, B, topk = 3000, 4, 256, 3
    kv_heads = 2 if layout == "gqa_head_major" else heads
    q, _, _, do, cu, mx = make_case(3, seqlen, heads, seed=21)
    _, k, v, _, _, _ = make_case(3, seqlen, kv_heads, seed=22)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    op = moba_attn_varlen_gqa if kv_heads != heads else moba_attn_varlen
    in_place = True
    if layout == "qkv_slices":
        base = torch.stack([q, k, v], dim=1).cuda().requires_grad_(True)       # [S, 3, H, D]
        views = [base[:, 0], base[:, 1], base[:, 2]]
    elif layout in ("head_major", "gqa_head_major"):
        leaves = [x.cuda().transpose(0, 1).contiguous().requires_grad_(True) for x in (q, k, v)]   # [H, S, D]
        views = [x.transpose(0, 1) for x in leaves]
    elif layout == "mixed":   # k token-major, v head-major: their strides differ, so both are copied
        leaves = [q.cuda().requires_grad_(True), k.cuda().requires_grad_(True),
                  v.cuda().transpose(0, 1).contiguous().requires_grad_(True)]
        views = [leaves[0], leaves[1], leaves[2].transpose(0, 1)]
    else:                     # rows that start 8 bytes into a 16-byte line
        leaves = [torch.zeros(x.numel() + 4, dtype=x.dtype, device="cuda") for x in (q, k, v)]
        views = []
        for buf, x in zip(leaves, (q, k, v)):
            buf[4:].copy_(x.cuda().reshape(-1))
            views.append(buf[4:].view(x.shape).requires_grad_(True))
        in_place = False
    got = E._in_place(*views)
    if layout in ("qkv_slices", "head_major", "gqa_head_major"):
        assert all(a is b for a, b in zip(got, views))
    elif layout == "mixed":
        assert got[0] is views[0] and got[1].is_contiguous() and got[2].is_contiguous()
    else:
        assert not in_place and all(a.data_ptr() % 16 == 0 for a in got)

    out = op(views[0], views[1], views[2], cu_t, mx, B, topk)
    out.backward(do.cuda())
    qc, kc, vc = (x.cuda().requires_grad_(True) for x in (q, k, v))
    want = op(qc, kc, vc, cu_t, mx, B, topk)
    want.backward(do.cuda())
    assert out.is_contiguous() and torch.equal(out, want)
    if layout == "qkv_slices":
        grads = [base.grad[:, 0], base.grad[:, 1], base.grad[:, 2]]
    elif layout in ("head_major", "gqa_head_major"):
        grads = [x.grad.transpose(0, 1) for x in leaves]
    elif layout == "mixed":
        grads = [leaves[0].grad, leaves[1].grad, leaves[2].grad.transpose(0, 1)]
    else:
        grads = [x.grad for x in views]
    for g, w in zip(grads, (qc.grad, kc.grad, vc.grad)):
        assert torch.equal(g, w)

    # the stages on their own
    from moba_amd.plan import make_plan
    plan = make_plan(cu_t, B, topk)
    kbar = E.chunk_mean(views[1].detach(), plan)
    assert torch.equal(kbar, E.chunk_mean(kc.detach(), plan))
    assert torch.equal(E.gate_topk(views[0].detach(), kbar, plan), E.gate_topk(qc.detach(), kbar, plan))


def test_more_than_64_history_chunks_is_refused():
    """The selection kernel keeps at most 64 candidates per row: a larger k is an error, not a wrong answer."""
    from moba_amd import moba_attn_varlen
    q, k, v, _, cu, mx = make_case(1, 4096, 1, seed=3)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="moba_gate_topk"):
        moba_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu_t, mx, 32, 80)
    out = moba_attn_varlen(q.cuda(), k.cuda(), v.cuda(), cu_t, mx, 32, 65)   # k = 64 is the last one served
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("b,hq,hkv,s,B,topk,dtype", [
    (3, 4, 2, 1500, 128, 3, torch.bfloat16),
    (2, 8, 8, 2048, 256, 4, torch.float16),
    (4, 4, 1, 700, 100, 2, torch.bfloat16),
    (2, 2, 2, 1024, 2048, 3, torch.bfloat16),      # one chunk per sequence: full causal attention
])
def test_batched_layout_in_place(b, hq, hkv, s, B, topk, dtype):
    """[batch, heads, seqlen, head_dim] tensors (the transformers layout) are read where they lie -- no transposing
    copies for batch > 1 -- and give bit for bit the output and the gradients of the packed operator on the copies
    hf_to_fa makes (moba/wrapper.py:7-15, :56-58); the packed operator itself is checked against the oracle."""
    from moba_amd import moba_attn_varlen, moba_attn_varlen_gqa
    from moba_amd import moba_efficient as E
    from moba_amd.wrapper import hf_to_fa
    g = torch.Generator().manual_seed(31)
    query = torch.randn((b, hq, s, 128), generator=g).to(dtype).cuda().requires_grad_(True)
    key = torch.randn((b, hkv, s, 128), generator=g).to(dtype).cuda().requires_grad_(True)
    value = torch.randn((b, hkv, s, 128), generator=g).to(dtype).cuda().requires_grad_(True)
    do = torch.randn((b * s, hq, 128), generator=g).to(dtype).cuda()
    assert E._addressable(query) and E._addressable(key) and E._strides(query, key)[4] == s
    out = E.moba_attn_batched(query, key, value, B, topk)
    out.backward(do)
    qp, kp, vp = (hf_to_fa(x.detach()).contiguous().requires_grad_(True) for x in (query, key, value))
    cu = torch.arange(0, (b + 1) * s, s, dtype=torch.int32, device="cuda")
    want = moba_attn_varlen_gqa(qp, kp, vp, cu, s, B, topk)
    want.backward(do)
    assert out.shape == (b * s, hq, 128) and torch.equal(out, want)
    for got, ref in ((query.grad, qp.grad), (key.grad, kp.grad), (value.grad, vp.grad)):
        assert got.shape[0] == b and torch.equal(hf_to_fa(got), ref)
    # and the oracle, on the packed copies with expanded key/value heads
    rep = hq // hkv
    cu_l = cu.tolist()
    from moba_amd.plan import make_plan
    plan = make_plan(cu, B, topk)
    sel = None if plan.fallback else E.gate_topk(qp.detach(), E.chunk_mean(kp.detach(), plan), plan).cpu()
    ref = O.moba_attn_varlen_oracle(qp.detach().cpu(), torch.repeat_interleave(kp.detach().cpu(), rep, dim=1),
                                    torch.repeat_interleave(vp.detach().cpu(), rep, dim=1), cu_l, s, B, topk, sel=sel)
    err = (out.detach().cpu().float() - ref).abs()
    assert err.max() < MAX_ABS and err.mean() < MEAN_ABS, (err.max().item(), err.mean().item())
    # a layout the kernels cannot address (rows 8 bytes off a 16-byte line) takes the copying path, same result
    buf = torch.zeros(query.numel() + 4, dtype=dtype, device="cuda")
    buf[4:].copy_(query.detach().reshape(-1))
    odd = buf[4:].view(query.shape)
    assert not E._addressable(odd)
    assert torch.equal(E.moba_attn_batched(odd, key.detach(), value.detach(), B, topk), want)


@pytest.mark.parametrize("heads,kv_heads,batched", [(6, 6, False), (8, 2, False), (8, 4, True), (10, 5, False)])
def test_heads_in_groups(heads, kv_heads, batched, monkeypatch):
    """A call whose per-slot partials would not fit its scratch budget (or 2^31 slot rows) works through its heads in
    groups of whole key/value head groups: same output, LSE and gradients bit for bit as in one piece -- the packed
    operator, grouped-query heads, and the batched layout read in place."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    from moba_amd.wrapper import hf_to_fa
    b, s, B, topk = 3, 1400, 128, 3
    g = torch.Generator().manual_seed(17)
    query = torch.randn((b, heads, s, 128), generator=g).to(torch.bfloat16).cuda()
    key = torch.randn((b, kv_heads, s, 128), generator=g).to(torch.bfloat16).cuda()
    value = torch.randn((b, kv_heads, s, 128), generator=g).to(torch.bfloat16).cuda()
    do = torch.randn((b * s, heads, 128), generator=g).to(torch.bfloat16).cuda()
    cu = torch.arange(0, (b + 1) * s, s, dtype=torch.int32, device="cuda")

    def run():
        if batched:
            q, k, v = (x.clone().requires_grad_(True) for x in (query, key, value))
            out = E.moba_attn_batched(q, k, v, B, topk)
        else:
            q, k, v = (hf_to_fa(x).contiguous().requires_grad_(True) for x in (query, key, value))
            out = E.moba_attn_varlen_gqa(q, k, v, cu, s, B, topk)
        out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad

    whole = run()
    plan = make_plan(cu, B, topk)
    rep = heads // kv_heads
    per_head = plan.S * (plan.K + 1) * (128 * 2 + 4)
    monkeypatch.setattr(E, "SCRATCH_LIMIT_BYTES", per_head * rep * 2 - 1)     # one key/value head group at a time
    assert E._head_groups(plan, heads, kv_heads, 128, 2) == [(h, h + rep) for h in range(0, heads, rep)]
    parts = run()
    for a, b_ in zip(whole, parts):
        assert a.shape == b_.shape and torch.equal(a, b_)
    if kv_heads > 2:
        monkeypatch.setattr(E, "SCRATCH_LIMIT_BYTES", per_head * rep * 3 - 1)     # two key/value heads at a time
        groups = E._head_groups(plan, heads, kv_heads, 128, 2)
        assert len(groups) == -(-kv_heads // 2) and groups[0] == (0, 2 * rep) and groups[-1][1] == heads
        assert all(a % rep == 0 and 0 < b_ - a <= 2 * rep for a, b_ in groups)
        for a, b_ in zip(whole, run()):
            assert torch.equal(a, b_)
    # the forward alone (no autograd)
    monkeypatch.setattr(E, "SCRATCH_LIMIT_BYTES", per_head * rep * 2 - 1)
    with torch.no_grad():
        q, k, v = (hf_to_fa(x).contiguous() for x in (query, key, value))
        out, lse = E.moba_attn_varlen_with_lse(q, k, v, cu, s, B, topk, gqa=True)
    assert torch.equal(out, whole[0])
