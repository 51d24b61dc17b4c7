"""All-rows parity of the kernels that large problems run: the forward kernel whose resident workgroups draw
tiles from the per-XCD queues (fixed-reference softmax plus its redo list, bf16 and fp16)
and the backward kernels with eight queues and the draw a tile ahead, with and without dense prefixes.  The
shapes are large enough for those forms and small enough for the dense-mask fp32 oracle, which runs one
sequence at a time.  Contract and tolerances: the reference's tests/test_moba_attn.py:37-100."""

import numpy as np
import pytest
import torch

from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3
REF_MAX_ABS, REF_MEAN_ABS = 4e-2, 4e-4
LENGTHS = [8155, 7777, 8192, 6013, 8000, 8492, 5000, 7919]   # none a multiple of the chunk but one


def oracle_by_sequence(q, k, v, do, cu, B, topk, sel):
    """out, lse, dq, dk, dv of the fp32 oracle on the given selection, one sequence at a time (the dense mask of
    a sequence is [heads, L, L])."""
    meta = O.calc_chunks(cu, B)
    parts = []
    for b in range(len(cu) - 1):
        s0, s1 = cu[b], cu[b + 1]
        qs, ks, vs = (x[s0:s1].clone().requires_grad_(True) for x in (q, k, v))
        sel_b = sel[s0:s1]
        sel_b = torch.where(sel_b >= 0, sel_b - int(meta["first_filtered"][b]), sel_b)
        out, lse, _ = O.moba_attn_varlen_oracle(qs, ks, vs, [0, s1 - s0], s1 - s0, B, topk, sel=sel_b, return_aux=True)
        out.backward(do[s0:s1].float())
        parts.append((out.detach(), lse.detach(), qs.grad, ks.grad, vs.grad))
    return tuple(torch.cat([p[i] for p in parts], dim=0) for i in range(5))


@pytest.mark.parametrize("dense,dtype,spread", [
    (True, torch.bfloat16, 1.0),     # what the operator picks for a problem of this size
    (False, torch.bfloat16, 1.0),    # the reference's own decomposition on the same kernels
    (True, torch.bfloat16, 8.0),     # near one-hot rows: tiles leave the fixed reference's range and are computed again
    (False, torch.bfloat16, 8.0),
    (True, torch.float16, 1.0),
    (False, torch.float16, 1.0),
    (True, torch.float16, 8.0),      # fp16 probabilities leave their range much sooner: many tiles computed again
])
def test_queued_kernels_against_the_dense_oracle(dense, dtype, spread, monkeypatch):
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    from moba_amd.plan import FWD_TILE_ROWS, TILE_ROWS, make_plan
    H, B, topk = 4, 512, 4
    cu = [0] + np.cumsum(LENGTHS).tolist()
    S = cu[-1]
    print("queued case", dense, dtype, spread, S, flush=True)
    g = torch.Generator().manual_seed(41)
    q, k, v, do = (torch.randn((S, H, 128), generator=g) for _ in range(4))
    q, k, v, do = (q * spread).to(dtype), (k * spread).to(dtype), v.to(dtype), do.to(dtype)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    monkeypatch.setattr(E, "DENSE_PREFIX", dense)
    monkeypatch.setattr(E, "KEEP_SCRATCH", True)
    base = make_plan(cu_t, B, topk)
    plan = E._choose_plan(base, H)
    assert plan.dense_local == (base.K if dense else 0)
    lib = _lib.load()
    # the forms under test: resident workgroups in the forward, eight queues and the look-ahead draw in the backward
    assert lib.moba_fwd_is_queued(plan.hist_tile_bound(H, FWD_TILE_ROWS), plan.fwd_self_tiles, H) == 1
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert plan.hist_tile_bound(H, TILE_ROWS) + plan.self_tiles * H >= 8 * 2 * ((cus + 7) // 8 * 8) or \
        "MOBA_RESIDENT_CUS" in __import__("os").environ

    qg, kg, vg = (x.cuda().requires_grad_(True) for x in (q, k, v))
    out, lse = E.moba_attn_varlen_with_lse(qg, kg, vg, cu_t, max(LENGTHS), B, topk)
    redo = E.last_scratch["redo"]
    n_redo = None if redo is None else int(redo[0])
    print("  tiles computed again:", n_redo, flush=True)
    assert n_redo is not None and ((n_redo == 0) if spread == 1.0 else (n_redo > 50))
    out.backward(do.cuda())

    # the selection: the gate's own (on the batch's plain plan), equal to the oracle's up to near-ties of the scores
    sel = E.gate_topk(qg.detach(), E.chunk_mean(kg.detach(), base), base).cpu()
    gate = O.gate_scores(q, O.chunk_mean(k, cu, B), cu, B)
    want = O.select_topk(gate, base.K)
    got = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got = torch.where(got == 1 << 30, torch.full_like(got, -1), got)
    diff_rows = (got != want).any(dim=-1)
    for s_, h_ in diff_rows.nonzero().tolist():
        a, b = set(got[s_, h_].tolist()) - {-1}, set(want[s_, h_].tolist()) - {-1}
        gap = max(abs(float(gate[s_, h_, x]) - float(gate[s_, h_, y])) for x in a ^ b for y in a ^ b)
        assert gap < 1e-4 * spread * spread, (s_, h_, a, b, gap)
    assert diff_rows.float().mean() < 1e-3

    ref, ref_lse, rdq, rdk, rdv = oracle_by_sequence(q, k, v, do, cu, B, topk, sel)
    err = (out.detach().cpu().float() - ref).abs()
    print("  out max", err.max().item(), "mean", err.mean().item(), flush=True)
    peaked = spread > 1.0
    assert err.max() < (3e-2 if peaked else MAX_ABS) and err.mean() < MEAN_ABS, (err.max().item(), err.mean().item())
    assert (lse.cpu() - ref_lse).abs().max() < 2e-3 * spread * spread
    if not peaked:
        err16 = (out.detach().cpu().float() - ref.to(dtype).float()).abs()
        assert err16.max() < REF_MAX_ABS and err16.mean() < REF_MEAN_ABS, (err16.max().item(), err16.mean().item())
    for name, got_g, want_g in (("dq", qg.grad, rdq), ("dk", kg.grad, rdk), ("dv", vg.grad, rdv)):
        e = (got_g.cpu().float() - want_g).abs()
        scale = want_g.abs().max().clamp_min(1.0)
        print("  ", name, "max", e.max().item(), "mean", e.mean().item(), "scale", scale.item(), flush=True)
        assert torch.isfinite(got_g.float()).all()
        if peaked:
            assert e.max() < 3e-2 * scale and e.mean() < 2e-2 * want_g.abs().mean() + 1e-4, name
        else:
            assert e.max() < MAX_ABS * scale and e.mean() < REF_MEAN_ABS, name
