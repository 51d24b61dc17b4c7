"""Stage-level parity of the HIP kernels against the CPU oracle (GPU only).
Everything is called through the C ABI of libmoba_hip.so via moba_amd."""

import numpy as np
import pytest
import torch

from conftest import make_case
from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu


def _plan(cu, B, topk, dense=False):
    from moba_amd.plan import make_plan
    plan = make_plan(torch.tensor(cu, dtype=torch.int32, device="cuda"), B, topk)
    return plan.with_dense_prefix() if dense else plan


def _token_chunk_local(cu, B):
    """index, inside its sequence, of the chunk of every token"""
    return torch.cat([torch.arange(b - a) // B for a, b in zip(cu[:-1], cu[1:])])


def _note(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ chunk mean
@pytest.mark.parametrize("batch,seqlen,heads,B", [(1, 2048, 4, 256), (4, 2048, 2, 128), (7, 1024, 8, 128),
                                                   (3, 3000, 3, 100), (1, 8192, 32, 1024)])
def test_chunk_mean_bit_exact(batch, seqlen, heads, B):
    from moba_amd import moba_efficient as E
    _note("chunk_mean", batch, seqlen, heads, B)
    q, k, v, _, cu, _ = make_case(batch, seqlen, heads, seed=1)
    plan = _plan(cu, B, 3)
    if plan.fallback:
        pytest.skip("no filtered chunk")
    got = E.chunk_mean(k.cuda(), plan).cpu()
    want = O.chunk_mean(k, cu, B)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_chunk_mean_rounds_once():
    """Means just above, just below and on a tie of the element type (see the oracle's test of the same name):
    the kernel rounds the fp64 mean once."""
    from moba_amd import moba_efficient as E
    for dtype, step, tiny in ((torch.bfloat16, 2.0 ** -7, 2.0 ** -38), (torch.float16, 2.0 ** -10, 2.0 ** -24)):
        k = torch.zeros((8, 1, 128), dtype=dtype)
        k[0, 0, :] = 4.0
        k[1, 0, 0] = 2 * step; k[2, 0, 0] = tiny
        k[1, 0, 1] = 2 * step; k[2, 0, 1] = -tiny
        k[1, 0, 2] = 2 * step
        k[1, 0, 3] = 6 * step
        plan = _plan([0, 8], 4, 2)
        got = E.chunk_mean(k.cuda(), plan).cpu()
        assert torch.equal(got, O.chunk_mean(k, [0, 8], 4))
        assert got[0, 0, 0].item() == 1 + step and got[0, 0, 1].item() == 1.0 and got[0, 0, 3].item() == 1 + 2 * step


def test_chunk_mean_exact_integers():
    from moba_amd import moba_efficient as E
    g = torch.Generator().manual_seed(2)
    k = torch.randint(-16, 17, (1024, 2, 128), generator=g).to(torch.bfloat16)
    cu = [0, 1024]
    plan = _plan(cu, 64, 3)
    got = E.chunk_mean(k.cuda(), plan).cpu().float()
    want = torch.stack([k[i * 64:(i + 1) * 64].float().sum(0) / 64 for i in range(15)]).to(torch.bfloat16).float()
    assert torch.equal(got, want)


# ------------------------------------------------------------------ gate + top-k
@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [(1, 2048, 4, 128, 3), (4, 2048, 2, 128, 4),
                                                        (7, 2048, 5, 64, 2), (2, 4096, 1, 32, 13),
                                                        (3, 1500, 3, 100, 3)])
def test_gate_scores_and_selection(batch, seqlen, heads, B, topk):
    from moba_amd import moba_efficient as E
    _note("gate", batch, seqlen, heads, B, topk)
    q, k, v, _, cu, _ = make_case(batch, seqlen, heads, seed=3)
    plan = _plan(cu, B, topk)
    kbar = O.chunk_mean(k, cu, B)
    sel, scores = E.gate_topk(q.cuda(), kbar.cuda(), plan, return_scores=True)
    sel, scores = sel.cpu(), scores.cpu()
    want = O.gate_scores(q, kbar, cu, B)
    # same -inf pattern; fp32 values differ only by summation order
    assert torch.equal(torch.isinf(scores), torch.isinf(want))
    fin = ~torch.isinf(want)
    assert (scores[fin] - want[fin]).abs().max() < 1e-4
    # selection is bit exact given the kernel's own scores
    want_sel = O.select_topk(scores, plan.K)
    got_sel = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got_sel = torch.where(got_sel == 1 << 30, torch.full_like(got_sel, -1), got_sel)
    assert torch.equal(got_sel, want_sel)
    # the call that writes no scores (the operator's; beyond 32 candidates it inserts only the candidates that
    # beat a list's worst entry) returns the same lists, order included
    assert torch.equal(E.gate_topk(q.cuda(), kbar.cuda(), plan).cpu(), sel)


@pytest.mark.parametrize("topk", [2, 4, 9, 13])
def test_gate_many_candidates_with_ties(topk):
    """Keys drawn from a handful of values and identical within runs of chunks: equal scores across and inside the
    blocks of 32 candidates.  The lists with and without the score output agree entry by entry, and equal the
    oracle's selection on the kernel's scores (lower chunk id first among equals)."""
    from moba_amd import moba_efficient as E
    S, H, B = 16384, 3, 64                      # 256 chunks: up to eight blocks of candidates per token
    g = torch.Generator().manual_seed(100 + topk)
    q = torch.randint(-2, 3, (S, H, 128), generator=g).to(torch.bfloat16)
    kc = torch.randint(-1, 2, (S // B // 4, 1, H, 128), generator=g).to(torch.bfloat16)
    k = kc.expand(-1, 4 * B, -1, -1).reshape(S, H, 128).contiguous()   # four consecutive chunks share their keys
    cu = [0, S]
    plan = _plan(cu, B, topk)
    kbar = E.chunk_mean(k.cuda(), plan)
    sel, scores = E.gate_topk(q.cuda(), kbar, plan, return_scores=True)
    plain = E.gate_topk(q.cuda(), kbar, plan)
    assert torch.equal(plain, sel)
    sel, scores = sel.cpu(), scores.cpu()
    fin = scores[torch.isfinite(scores)]
    assert fin.numel() > 0 and fin.unique().numel() < fin.numel() // 100      # ties everywhere
    want_sel = O.select_topk(scores, plan.K)
    got_sel = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got_sel = torch.where(got_sel == 1 << 30, torch.full_like(got_sel, -1), got_sel)
    assert torch.equal(got_sel, want_sel)
    # descending score, ascending id among equal scores, along every list
    sc = torch.gather(scores, 2, sel.clamp_min(0).long())
    sc = torch.where(sel >= 0, sc, torch.full_like(sc, float("-inf")))
    assert bool((sc[..., 1:] <= sc[..., :-1]).all())
    same = (sc[..., 1:] == sc[..., :-1]) & (sel[..., 1:] >= 0)
    assert bool((sel[..., 1:][same] > sel[..., :-1][same]).all())


@pytest.mark.parametrize("K", [1, 2, 3, 5, 11, 16, 40])
def test_topk_from_injected_scores_bit_exact(K):
    from moba_amd import moba_efficient as E
    g = torch.Generator().manual_seed(K)
    S, H, F = 300, 3, 77
    scores = torch.randn((S, H, F), generator=g)
    # ties, -inf runs and rows with fewer than K candidates
    scores[:, :, ::7] = scores[:, :, 1::7][:, :, :scores[:, :, ::7].shape[-1]]
    scores[::3, :, 20:] = float("-inf")
    scores[5::11] = float("-inf")
    scores[7, 0, :] = 1.0
    sel = E.topk_from_scores(scores.cuda(), K).cpu()
    got = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got = torch.where(got == 1 << 30, torch.full_like(got, -1), got)
    assert torch.equal(got, O.select_topk(scores, K))
    # the kernel's own order is descending score, ties by ascending id
    assert sel[7, 0].tolist() == list(range(min(K, F)))


# ------------------------------------------------------------------ gather lists
# (the last cases: more candidate chunks than one pass of the gate's LDS histogram holds; more chunks in a
# sequence than the list fill's four-wave form has LDS for)
@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("counted", [False, True])
@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [(1, 2048, 2, 128, 3), (5, 3000, 3, 100, 4), (2, 9000, 1, 64, 12),
                                                       (3, 5000, 5, 192, 2), (1, 140817, 1, 64, 2),
                                                       (1, 60007, 2, 16, 3)])
def test_gather_lists(batch, seqlen, heads, B, topk, counted, dense):
    """The lists from the counting pass of moba_build_lists, and from the counts the gate leaves as a by-product
    in an array that the chunk mean cleared.  With dense prefixes the tokens of the first K + 1 chunks of every
    sequence have no picks and no list entries; every other token's picks are what they are without."""
    from moba_amd import moba_efficient as E
    _note("lists", batch, seqlen, heads, B, topk, counted, dense)
    q, k, v, _, cu, _ = make_case(batch, seqlen, heads, seed=4)
    plan = _plan(cu, B, topk, dense)
    kbar = O.chunk_mean(k, cu, B)
    if dense:
        plain = E.gate_topk(q.cuda(), kbar.cuda(), _plan(cu, B, topk)).cpu()
        in_prefix = (_token_chunk_local(cu, B) <= plan.K)[:, None, None].expand_as(plain)
        want_sel = torch.where(in_prefix, torch.full_like(plain, -1), plain)
        assert plan.dense_local == plan.K > 0 and bool(in_prefix.any())
        assert torch.equal(E.gate_topk(q.cuda(), kbar.cuda(), plan).cpu(), want_sel)
    if counted:
        buffers = E.list_buffers(plan, heads, torch.device("cuda"))
        for b in buffers:
            b.fill_(0x5A5A5A5A)
        assert torch.equal(E.chunk_mean(k.cuda(), plan, clear=buffers[0]).cpu(), kbar)
        assert int(buffers[0].abs().max()) == 0 and int(buffers[1][0]) == 0x5A5A5A5A
        sel = E.gate_topk(q.cuda(), kbar.cuda(), plan, cnt=buffers[0])
        assert int(buffers[0].sum()) == plan.pairs_per_head * heads
        assert torch.equal(sel, E.gate_topk(q.cuda(), kbar.cuda(), plan))
        lists = E.build_lists(sel, plan, buffers=buffers, counted=True, second_tile_rows=128)
    else:
        sel = E.gate_topk(q.cuda(), kbar.cuda(), plan)
        lists = E.build_lists(sel, plan, second_tile_rows=128)
    seg_off, tile_off, seg_dest, tile_seg, second_off, second_seg = (x.cpu().numpy() for x in lists)
    sel = sel.cpu()
    counts, offs, rows, slots = O.gather_lists(sel, plan.F)
    H, K1 = heads, plan.K + 1
    assert offs[-1] == plan.pairs_per_head * H
    if not dense:
        assert offs[-1] == O.expected_pair_count(cu, B, plan.K, H)
    assert np.array_equal(seg_off, offs)
    heads_of = np.repeat(np.arange(plan.F * H) % H, counts)
    want_dest = (rows * H + heads_of) * K1 + 1 + slots
    assert np.array_equal(seg_dest[:offs[-1]], want_dest)
    from moba_amd import _lib
    lib = _lib.load()
    fwd_rows, bwd_rows = lib.moba_fwd_tile_rows(), lib.moba_bwd_tile_rows()
    assert (fwd_rows, bwd_rows) == (256, 128)
    # the tile tables: the forward kernel's from moba_build_lists, the backward kernels' from moba_tile_tables
    bwd_off, bwd_seg = (x.cpu().numpy() for x in E.tile_tables(torch.from_numpy(seg_off).cuda(), plan, H, bwd_rows))
    # ... or, for a caller that asks, from moba_build_lists as a second pair
    assert np.array_equal(second_off, bwd_off) and np.array_equal(second_seg, bwd_seg)
    for rows_per_tile, toff, tseg in ((fwd_rows, tile_off, tile_seg), (bwd_rows, bwd_off, bwd_seg)):
        tiles = (counts + rows_per_tile - 1) // rows_per_tile
        assert np.array_equal(toff, np.concatenate([[0], np.cumsum(tiles)]))
        # every history tile id names its segment; ids past the last tile are marked
        want_seg = np.repeat(np.arange(plan.F * H), tiles)
        assert tseg.size == plan.hist_tile_bound(H, rows_per_tile) >= want_seg.size
        assert np.array_equal(tseg[:want_seg.size], want_seg) and (tseg[want_seg.size:] == -1).all()


# ------------------------------------------------------------------ forward
@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [
    (1, 1024, 2, 128, 3), (4, 2048, 4, 256, 2), (7, 2048, 1, 128, 4), (3, 1500, 3, 100, 3),
    (1, 512, 2, 1024, 3), (2, 4096, 2, 64, 12), (1, 2048, 2, 128, 1)])
def test_forward_vs_oracle(batch, seqlen, heads, B, topk):
    from moba_amd import moba_efficient as E
    _note("fwd", batch, seqlen, heads, B, topk)
    q, k, v, _, cu, mx = make_case(batch, seqlen, heads, seed=5)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    plan = _plan(cu, B, topk)
    out, lse = E.moba_attn_varlen_with_lse(q.cuda(), k.cuda(), v.cuda(), cu_t, mx, B, topk)
    out, lse = out.cpu().float(), lse.cpu()
    sel = None
    if not plan.fallback:
        kbar = E.chunk_mean(k.cuda(), plan)
        sel = E.gate_topk(q.cuda(), kbar, plan).cpu()
    want, want_lse, _ = O.moba_attn_varlen_oracle(q, k, v, cu, mx, B, topk, sel=sel, return_aux=True)
    err = (out - want).abs()
    _note("  max", err.max().item(), "mean", err.mean().item(), "lse", (lse - want_lse).abs().max().item())
    assert err.max() < 2e-2 and err.mean() < 2e-3           # the stated bf16 tolerance
    assert err.mean() < 4e-4                                 # the reference test's own mean bound
    assert (lse - want_lse).abs().max() < 2e-3


# ------------------------------------------------------------------ LSE merge alone
@pytest.mark.parametrize("K,dtype,parts", [(2, torch.bfloat16, 1), (11, torch.bfloat16, 1), (20, torch.float16, 1),
                                           (3, torch.bfloat16, 2), (17, torch.float16, 4)])
def test_merge_of_random_partials(K, dtype, parts):
    """moba_fwd_merge on random per-slot partials (some slots absent, log-sum-exps far apart)
    against the merge algebra of the oracle (moba/moba_efficient.py:130-168).  parts > 1: every history slot
    holds that many partials (key_split of the forward), the self slot one."""
    import ctypes
    import math
    from moba_amd import _lib
    lib = _lib.load()
    S, H, K1 = 300, 3, K + 1
    g = torch.Generator().manual_seed(K)
    part_o = torch.randn((parts, S * H * K1, 128), generator=g).to(dtype)
    lse_nat = torch.randn((parts, S * H, K1), generator=g) * 6             # natural-log LSE of each slot
    sel = torch.randint(0, 50, (S, H, K), generator=g, dtype=torch.int32)
    sel[torch.rand((S, H, K), generator=g) < 0.3] = -1                     # absent slots
    part_o_dev = part_o.cuda()
    # absent slots hold garbage in the real buffers (and so do parts 1.. of the self slot): poison them
    absent = torch.cat([torch.zeros((S * H, 1), dtype=torch.bool), (sel < 0).view(S * H, K)], dim=1)
    absent = absent.unsqueeze(0).repeat(parts, 1, 1)
    absent[1:, :, 0] = True
    part_o_dev.view(parts, S * H, K1, 128)[absent.cuda()] = float("nan")
    part_lse = (lse_nat / math.log(2.0)).float()                           # the kernels keep it in the log2 domain
    part_lse_dev = part_lse.clone()
    part_lse_dev[absent] = float("nan")
    part_lse_dev = part_lse_dev.view(-1).cuda()
    out = torch.empty((S, H, 128), dtype=dtype, device="cuda")
    lse = torch.empty((S, H), dtype=torch.float32, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    code = _lib.DTYPE_F16 if dtype == torch.float16 else _lib.DTYPE_BF16
    _lib.check(lib.moba_fwd_merge(p(part_o_dev), p(part_lse_dev), p(sel.cuda()), p(out), p(lse), S, H, 128, K, parts,
                                  None, None, 0, S, code, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)),
               "moba_fwd_merge")
    lses = lse_nat.clone()
    lses[absent] = float("-inf")
    # (the parts of a slot are slots like any other to the merge algebra)
    want, want_lse = O.merge_partials(part_o.float().view(parts, S * H, K1, 128).permute(0, 2, 1, 3).reshape(parts * K1, S * H, 128),
                                      lses.permute(0, 2, 1).reshape(parts * K1, S * H))
    assert (out.float().cpu().view(S * H, 128) - want).abs().max() < 2e-2
    assert (lse.cpu().view(-1) - want_lse).abs().max() < 1e-3


# ------------------------------------------------------------------ the one-call attention entry point
@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("batch,seqlen,heads,B,topk,dtype", [(3, 3000, 3, 100, 3, torch.bfloat16),
                                                              (2, 4096, 2, 256, 4, torch.float16),
                                                              (1, 2048, 2, 128, 1, torch.bfloat16)])
def test_moba_fwd_entry_point(batch, seqlen, heads, B, topk, dtype, dense):
    """moba_fwd (partial attentions + merge behind one call): bit for bit what moba_fwd_partials followed by
    moba_fwd_merge give, and within the tolerances of the oracle run on the same selection (with dense prefixes:
    on the selection of the plain plan, whose attended sets are the same)."""
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    _note("moba_fwd", batch, seqlen, heads, B, topk, dtype, dense)
    q, k, v, _, cu, mx = make_case(batch, seqlen, heads, seed=9, dtype=dtype)
    plan = _plan(cu, B, topk, dense)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    want_out, want_lse, sel, seg_off, tile_off, seg_dest, tile_seg = E._forward(qg, kg, vg, plan)
    lib = _lib.load()
    S, H, D = q.shape
    K, t, dev = plan.K, plan.tables, qg.device
    bound = plan.hist_tile_bound(H, 256)
    split = 1 if plan.fallback else lib.moba_fwd_key_split(S, H, K, plan.chunk_size, bound, plan.fwd_self_tiles)  # as the operator
    part_o = torch.empty((split * S * H * (K + 1), D), dtype=dtype, device=dev)
    part_lse = torch.empty((split * S * H * (K + 1),), dtype=torch.float32, device=dev)
    out = torch.zeros((S, H, D), dtype=dtype, device=dev)
    lse = torch.zeros((S, H), dtype=torch.float32, device=dev)
    queues = torch.empty(8, dtype=torch.int32, device=dev)
    p = E._ptr
    _lib.check(lib.moba_fwd(p(qg), p(kg), p(vg), p(part_o), p(part_lse), p(sel), p(seg_off), p(tile_off), p(seg_dest),
                            p(t.get("fchunk_tok")), p(t["achunk_tok"]), p(t["fwd_self_tile_prefix"]), p(tile_seg),
                            p(t["fwd_self_tile_chunk"]), p(t["achunk_direct"]), p(t["mrg_start"]), p(t["mrg_prefix"]),
                            plan.nseq, plan.merge_tokens, p(out), p(lse), S, H, H, D, K, plan.F, plan.NA,
                            plan.chunk_size, bound, plan.fwd_self_tiles, split, None, p(queues), None, 0.0,
                            E._dtype_code(qg), E._stream(dev)), "moba_fwd")
    torch.cuda.synchronize()
    assert torch.equal(out, want_out) and torch.equal(lse, want_lse)
    if dense and sel is not None:
        sel = E.gate_topk(qg, E.chunk_mean(kg, plan), _plan(cu, B, topk))
    ref, ref_lse, _ = O.moba_attn_varlen_oracle(q, k, v, cu, mx, B, topk, sel=None if sel is None else sel.cpu(),
                                                return_aux=True)
    err = (out.cpu().float() - ref).abs()
    assert err.max() < 2e-2 and err.mean() < 2e-3, (err.max().item(), err.mean().item())
    assert (lse.cpu() - ref_lse).abs().max() < 2e-3


# ------------------------------------------------------------------ fixed-reference softmax and its redo list
def _attention_stage(q, k, v, plan, aux, with_redo, key_split=1, direct=True):
    """moba_fwd on prepared selection/lists; returns (out, lse, number of tiles sent to the redo list or None).
    direct: the rows without history slots go straight to the outputs (as the operator runs it), or every row
    through its slot and the merge."""
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    lib = _lib.load()
    sel, seg_off, tile_off, seg_dest, tile_seg = aux
    S, H, D = q.shape
    K, t, dev = plan.K, plan.tables, q.device
    # (poisoned: a part that the kernel does not write, or a slot the merge must not read, shows)
    part_o = torch.full((key_split * S * H * (K + 1), D), float("nan"), dtype=q.dtype, device=dev)
    part_lse = torch.full((key_split * S * H * (K + 1),), float("nan"), dtype=torch.float32, device=dev)
    out = torch.zeros((S, H, D), dtype=q.dtype, device=dev)
    lse = torch.zeros((S, H), dtype=torch.float32, device=dev)
    queues = torch.empty(8, dtype=torch.int32, device=dev)
    tiles = plan.hist_tile_bound(H, 256) + plan.fwd_self_tiles * H
    redo = torch.full((1 + tiles,), -7, dtype=torch.int32, device=dev) if with_redo else None
    p = E._ptr
    _lib.check(lib.moba_fwd(p(q), p(k), p(v), p(part_o), p(part_lse), p(sel), p(seg_off), p(tile_off), p(seg_dest),
                            p(t.get("fchunk_tok")), p(t["achunk_tok"]), p(t["fwd_self_tile_prefix"]), p(tile_seg),
                            p(t["fwd_self_tile_chunk"]), p(t["achunk_direct"]) if direct else None,
                            p(t["mrg_start"]) if direct else None, p(t["mrg_prefix"]) if direct else None,
                            plan.nseq if direct else 0, plan.merge_tokens if direct else S, p(out), p(lse), S, H, H, D, K,
                            plan.F, plan.NA, plan.chunk_size, plan.hist_tile_bound(H, 256), plan.fwd_self_tiles, key_split,
                            None, p(queues), p(redo), 0.0, E._dtype_code(q), E._stream(dev)), "moba_fwd")
    torch.cuda.synchronize()
    if redo is None:
        return out, lse, None
    n = int(redo[0])
    ids = redo[1:1 + n].cpu()
    assert 0 <= n <= tiles and ids.unique().numel() == n and bool(((ids >= 0) & (ids < tiles)).all())
    return out, lse, n


@pytest.mark.parametrize("seqlens,heads,B,topk,dtype", [([8192], 2, 1024, 3, torch.bfloat16),
                                                         ([3000, 5000, 777], 3, 512, 2, torch.float16),
                                                         ([16384], 1, 2048, 3, torch.bfloat16),
                                                         ([4000], 2, 192, 3, torch.bfloat16)])
def test_history_keys_cut_into_parts(seqlens, heads, B, topk, dtype):
    """key_split of moba_fwd: every history tile's keys in 2, 4 or 8 parts (tiles of their own whose partials the
    merge takes as further slots).  The result must agree with the uncut one within rounding and with the oracle
    on the same selection; what moba_fwd_key_split proposes must be accepted; values the call cannot serve are
    refused."""
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    lib = _lib.load()
    _note("key parts", seqlens, heads, B, topk, dtype)
    cu = [0] + [int(x) for x in np.cumsum(seqlens)]
    S = cu[-1]
    g = torch.Generator().manual_seed(sum(seqlens) + heads)
    q, k, v = (torch.randn((S, heads, 128), generator=g).to(dtype) for _ in range(3))
    plan = _plan(cu, B, topk)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    sel = E.gate_topk(qg, E.chunk_mean(kg, plan), plan)
    aux = (sel,) + tuple(E.build_lists(sel, plan))
    out1, lse1, _ = _attention_stage(qg, kg, vg, plan, aux, False, 1)
    # the rows without history slots written straight to the outputs, or through slot 0 and the merge: same bits
    out0, lse0, _ = _attention_stage(qg, kg, vg, plan, aux, False, 1, direct=False)
    assert torch.equal(out0, out1) and (lse0 - lse1).abs().max() < 1e-6
    ref, ref_lse, _ = O.moba_attn_varlen_oracle(q, k, v, cu, max(seqlens), B, topk, sel=sel.cpu(), return_aux=True)
    proposed = lib.moba_fwd_key_split(S, heads, plan.K, B, plan.hist_tile_bound(heads, 256), plan.fwd_self_tiles)
    _note("  proposed", proposed)
    assert proposed in (1, 2, 4, 8) and B % (64 * proposed) == 0
    for split in (2, 4, 8):
        if B % (64 * split):
            with pytest.raises(RuntimeError):
                _attention_stage(qg, kg, vg, plan, aux, False, split)
            continue
        out, lse, _ = _attention_stage(qg, kg, vg, plan, aux, False, split)
        assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
        d = (out.float() - out1.float()).abs()
        assert d.max() < 2e-2 and d.mean() < 2e-4, (split, d.max().item(), d.mean().item())
        assert (lse - lse1).abs().max() < 1e-3
        err = (out.cpu().float() - ref).abs()
        assert err.max() < 2e-2 and err.mean() < 2e-3, (split, err.max().item(), err.mean().item())
        assert (lse.cpu() - ref_lse).abs().max() < 2e-3
    for bad in (0, 3, 16):
        with pytest.raises(RuntimeError):
            _attention_stage(qg, kg, vg, plan, aux, False, bad)


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("spread", [1.0, 8.0])
def test_fixed_reference_softmax_and_redo_list(spread, dense):
    """A problem large enough for the resident-workgroup forward kernel (bf16): with a redo list the kernel takes
    each tile's softmax relative to a fixed per-row reference.  On N(0,1) data no tile leaves its range; with q
    and k scaled by 8 (logits of +-64 nats around zero, near one-hot rows) many do and are computed again by the
    kernel that tracks the maximum.  Either way the result must agree with the running-maximum path and with an
    explicit fp32 softmax over sampled rows' attended keys."""
    from moba_amd import moba_efficient as E
    from test_gpu_large import _row_oracle
    S, H, B, topk = 32768, 8, 1024, 3
    _note("fixed reference", S, H, B, topk, spread, dense)
    g = torch.Generator(device="cuda").manual_seed(17)
    q, k, v = (torch.randn((S, H, 128), generator=g, device="cuda", dtype=torch.float32) for _ in range(3))
    q, k, v = (q * spread).to(torch.bfloat16), (k * spread).to(torch.bfloat16), v.to(torch.bfloat16)
    plan = _plan([0, S], B, topk, dense)
    sel = E.gate_topk(q, E.chunk_mean(k, plan), plan)
    aux = (sel,) + tuple(E.build_lists(sel, plan))
    if dense:   # (the rows' attended sets, for the row oracle below: the plain plan's selection)
        sel = E.gate_topk(q, E.chunk_mean(k, plan), _plan([0, S], B, topk))
    out_f, lse_f, n_redo = _attention_stage(q, k, v, plan, aux, True)
    out_m, lse_m, _ = _attention_stage(q, k, v, plan, aux, False)
    _note("  tiles computed again:", n_redo)
    assert (n_redo == 0) if spread == 1.0 else (n_redo > 100)
    assert torch.isfinite(out_f.float()).all() and torch.isfinite(lse_f).all()
    err = (out_f.float() - out_m.float()).abs()
    assert err.max() < 2e-2 and err.mean() < 1e-4, (err.max().item(), err.mean().item())
    assert (lse_f - lse_m).abs().max() < 1e-3 * max(1.0, spread * spread)
    rng = np.random.default_rng(1)
    for s in sorted(set(rng.integers(0, S, size=24).tolist() + [0, S - 1, B, B - 1])):
        for h in (0, H - 1):
            ref, ref_lse = _row_oracle(q, k, v, sel[s, h].cpu(), s, h, 0, B, 0)
            e = (out_f[s, h].float().cpu() - ref).abs().max().item()
            assert e < 2e-2 and e <= 3e-2 * ref.abs().max().item() + 1e-5, (s, h, e)
            assert abs(lse_f[s, h].item() - ref_lse.item()) < 2e-3 * max(1.0, spread * spread)
    if spread == 1.0:  # the resident-workgroup kernel takes whole tiles only: key parts are refused, not ignored
        with pytest.raises(RuntimeError):
            _attention_stage(q, k, v, plan, aux, False, 2)
    else:
        # Values of large magnitude: probabilities of up to 2^96 times |v| of 2^40 leave fp32 in the accumulators of
        # the fixed-reference kernel, where the kernel that tracks the maximum (probabilities up to 2^8) stays
        # finite.  Such tiles must be found and computed again: the result is finite and the other path's.
        big = (v.float() * 2.0 ** 40).to(torch.bfloat16)
        out_b, lse_b, n_big = _attention_stage(q, k, big, plan, aux, True)
        out_r, lse_r, _ = _attention_stage(q, k, big, plan, aux, False)
        _note("  tiles computed again with |v| ~ 2^40:", n_big)
        assert n_big >= n_redo and torch.isfinite(out_b.float()).all() and torch.isfinite(out_r.float()).all()
        err = (out_b.float() - out_r.float()).abs() * 2.0 ** -40
        assert err.max() < 2e-2 and err.mean() < 1e-4, (err.max().item(), err.mean().item())
        assert torch.equal(lse_b, lse_f)
