"""Full-size configurations: the dense oracle cannot run there, so parity is checked on
sampled (token, head) rows against an explicit fp32 softmax over the row's attended keys,
and on size-independent properties of the selection and of the gather lists."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(S, H, Hkv, seed=0):
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(seed)
    q = torch.randn((S, H, 128), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    k = torch.randn((S, Hkv, 128), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    v = torch.randn((S, Hkv, 128), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    if Hkv != H:
        k = torch.repeat_interleave(k, H // Hkv, dim=1).contiguous()
        v = torch.repeat_interleave(v, H // Hkv, dim=1).contiguous()
    return q, k, v


def _row_oracle(q, k, v, sel_row, s, h, s0, B, fb):
    """fp32 attention of token s, head h over its own chunk (causal) and its selected chunks."""
    t = s - s0
    c = t // B
    idx = [torch.arange(s0 + c * B, s + 1)]
    for f in sel_row.tolist():
        if f >= 0:
            lc = f - fb
            idx.append(torch.arange(s0 + lc * B, s0 + (lc + 1) * B))
    idx = torch.cat(idx).to(q.device)
    kk = k[idx, h].float().cpu()
    vv = v[idx, h].float().cpu()
    qq = q[s, h].float().cpu()
    logits = (kk @ qq) * 128 ** -0.5
    lse = torch.logsumexp(logits, 0)
    return torch.exp(logits - lse) @ vv, lse


def _row_dq(q, k, v, dout, sel_row, s, h, s0, B, fb):
    """fp64 dq of token s, head h from the explicit softmax over its attended keys."""
    t = s - s0
    idx = [torch.arange(s0 + (t // B) * B, s + 1)]
    for f in sel_row.tolist():
        if f >= 0:
            idx.append(torch.arange(s0 + (f - fb) * B, s0 + (f - fb + 1) * B))
    idx = torch.cat(idx).to(q.device)
    kk, vv = k[idx, h].double().cpu(), v[idx, h].double().cpu()
    qq, do = q[s, h].double().cpu(), dout[s, h].double().cpu()
    scale = 128 ** -0.5
    p = torch.softmax(kk @ qq * scale, 0)
    dp = vv @ do
    ds = p * (dp - (p * dp).sum())
    return scale * (ds @ kk)


def _key_dkdv(q, k, v, out, lse, dout, sel, j, h, s0, s1, B, fb):
    """fp32 dk, dv of key j, head h: sums over every query that attends it, which are the later
    rows of its own chunk and the rows whose selection names its chunk.  Uses the forward's
    out and lse (checked separately) for the softmax statistics."""
    lc = (j - s0) // B
    own = torch.arange(j, min(s0 + (lc + 1) * B, s1), device=q.device)
    hist = torch.nonzero((sel[s0:s1, h] == fb + lc).any(-1)).flatten() + s0
    rows = torch.cat([own, hist])
    scale = 128 ** -0.5
    qq, do = q[rows, h].double(), dout[rows, h].double()
    p = torch.exp(qq @ k[j, h].double() * scale - lse[rows, h].double())
    delta = (out[rows, h].double() * do).sum(-1)
    ds = p * (do @ v[j, h].double() - delta)
    return (scale * (ds @ qq)).cpu(), (p @ do).cpu()


@pytest.mark.parametrize("lens,H,Hkv,B,topk", [
    ([131072], 32, 8, 4096, 12),                     # headline configuration
    ([59436, 29343, 53769, 62439, 31658, 6749, 21064, 37602], 32, 32, 2048, 3),   # varlen batch
    ([1048576], 32, 8, 4096, 12),                    # 1M tokens: largest index ranges
    ([32005, 777], 2, 2, 16, 3),                     # 2001 chunks in one sequence: the list builder's big-LDS path
    ([60007, 500], 2, 2, 16, 3),                     # 3751 chunks in one sequence: its one-wave form
    ([13001, 1, 26999, 300], 5, 5, 300, 5),          # odd everything, enough tiles for the tile queues
])
def test_sampled_rows_and_invariants(lens, H, Hkv, B, topk):
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan

    S = sum(lens)
    cu = np.concatenate([[0], np.cumsum(lens)])
    print("large case", S, H, B, topk, flush=True)
    q, k, v = _inputs(S, H, Hkv)
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    plan = make_plan(cu_t, B, topk)
    with_bwd = True                 # (at 1M tokens the per-slot partials of forward and backward, 103 GB each, share their memory)
    q.requires_grad_(with_bwd), k.requires_grad_(with_bwd), v.requires_grad_(with_bwd)
    out, lse = E.moba_attn_varlen_with_lse(q, k, v, cu_t, max(lens), B, topk)
    if with_bwd:
        g = torch.Generator(device="cuda").manual_seed(7)
        dout = torch.randn(out.shape, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
        dq, dk, dv = torch.autograd.grad(out, (q, k, v), dout)
    q, k, v, out = q.detach(), k.detach(), v.detach(), out.detach()
    kbar = E.chunk_mean(k, plan)
    sel = E.gate_topk(q, kbar, plan)
    seg_off, tile_off, seg_dest, tile_seg = E.build_lists(sel, plan)
    torch.cuda.synchronize()

    # ---- selection invariants over every row (on the GPU) ----
    tok = torch.arange(S, device="cuda")
    seq = torch.searchsorted(cu_t.long()[1:], tok, right=True)
    s0 = cu_t.long()[seq]
    c = (tok - s0) // B                                              # chunk index inside the sequence
    fb = plan.tables["seq_fbase"].long()[seq]
    nsel = (sel >= 0).sum(-1)                                        # [S, H]
    assert torch.equal(nsel, torch.minimum(c, torch.tensor(plan.K, device="cuda"))[:, None].expand(S, H))
    valid = sel >= 0
    lo = fb[:, None, None].expand_as(sel)
    hi = (fb + c)[:, None, None].expand_as(sel)
    assert bool((((sel >= lo) & (sel < hi)) | ~valid).all())         # strictly earlier chunks of the same sequence
    del lo, hi
    srt = torch.sort(torch.where(valid, sel, torch.full_like(sel, 1 << 30)), dim=-1).values
    assert not bool(((srt[..., 1:] == srt[..., :-1]) & (srt[..., 1:] < (1 << 30))).any())    # no chunk twice
    del srt
    # ---- gather lists: sizes and a checksum of the (token, head, slot) triples ----
    M = plan.pairs_per_head * H
    assert int(seg_off[-1]) == M == int(nsel.sum())
    K1 = plan.K + 1
    want = ((tok[:, None, None] * H + torch.arange(H, device="cuda")[None, :, None]) * K1 + 1
            + torch.arange(plan.K, device="cuda")[None, None, :])
    zero = torch.zeros((), dtype=torch.long, device="cuda")
    assert int(torch.where(valid, want, zero).sum()) == int(seg_dest[:M].long().sum())
    assert int(torch.where(valid, want * 7919 % 1000003, zero).sum()) == int((seg_dest[:M].long() * 7919 % 1000003).sum())
    # every list entry sits in the segment of the chunk it names
    seg_of = torch.searchsorted(seg_off.long()[1:], torch.arange(M, device="cuda"), right=True)
    d = seg_dest[:M].long()
    row, slot = d // K1, d % K1 - 1
    assert torch.equal(sel.view(-1, plan.K)[row, slot].long() * H + row % H, seg_of)
    del want, seg_of, d, row, slot

    # ---- sampled rows against the explicit softmax ----
    rng = np.random.default_rng(0)
    rows = sorted(set(rng.integers(0, S, size=14).tolist() + [0, S - 1, int(cu[1]) - 1, min(S - 1, B), min(S - 1, B - 1)]))
    worst = 0.0
    for s in rows:
        for h in sorted({0, min(H // 2 + 1, H - 1), H - 1}):
            b = int(np.searchsorted(cu, s, side="right") - 1)
            ref, ref_lse = _row_oracle(q, k, v, sel[s, h].cpu(), s, h, int(cu[b]), B, int(plan.host["seq_fbase"][b]))
            err = (out[s, h].float().cpu() - ref).abs().max().item()
            worst = max(worst, err)
            assert err < 2e-2, (s, h, err)
            assert err <= 3e-2 * ref.abs().max().item() + 1e-5, (s, h, err)
            assert abs(lse[s, h].item() - ref_lse.item()) < 2e-3
            if with_bwd:
                want_dq = _row_dq(q, k, v, dout, sel[s, h].cpu(), s, h, int(cu[b]), B, int(plan.host["seq_fbase"][b]))
                e = (dq[s, h].double().cpu() - want_dq).abs().max().item()
                assert e <= 2e-2 and e <= 3e-2 * want_dq.abs().max().item() + 1e-5, ("dq", s, h, e)
                fbq = int(plan.host["seq_fbase"][b])
                want_dk, want_dv = _key_dkdv(q, k, v, out, lse, dout, sel, s, h, int(cu[b]), int(cu[b + 1]), B, fbq)
                e = (dk[s, h].double().cpu() - want_dk).abs().max().item()
                assert e <= 2e-2 and e <= 3e-2 * want_dk.abs().max().item() + 1e-4, ("dk", s, h, e)
                e = (dv[s, h].double().cpu() - want_dv).abs().max().item()
                assert e <= 2e-2 and e <= 3e-2 * want_dv.abs().max().item() + 1e-4, ("dv", s, h, e)
    print("  worst sampled max-abs", worst, flush=True)


def test_chunk_mean_many_chunks():
    """More filtered chunks than a 16-bit grid dimension holds; exact against an fp64 mean."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    B, F, H = 8, 70000, 2
    S = B * (F + 1)
    g = torch.Generator(device="cuda").manual_seed(3)
    k = torch.randn((S, H, 128), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    plan = make_plan([0, S], B, 3, device="cuda")
    assert plan.F == F
    kbar = E.chunk_mean(k, plan)
    want = (k[:F * B].double().view(F, B, H, 128).sum(1) / B).float().to(torch.bfloat16)
    assert torch.equal(kbar, want)


def test_a_million_tokens_of_64_heads():
    """1M tokens x 64 query heads x top-k 12: 8.05e8 slot rows, 206 GB of per-slot partials in one piece.  The
    operator works through the heads in groups that fit its scratch budget (the reference has no such limit,
    moba/moba_efficient.py:270-297).  Forward, grouped-query heads (8 key/value heads), sampled rows against the
    explicit softmax over the row's attended keys."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    S, H, Hkv, B, topk = 1048576, 64, 8, 4096, 12
    print("large case", S, H, B, topk, flush=True)
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(5)
    q = torch.randn((S, H, 128), generator=g, device=dev, dtype=torch.bfloat16)
    k = torch.randn((S, Hkv, 128), generator=g, device=dev, dtype=torch.bfloat16)
    v = torch.randn((S, Hkv, 128), generator=g, device=dev, dtype=torch.bfloat16)
    cu_t = torch.tensor([0, S], dtype=torch.int32, device=dev)
    plan = make_plan(cu_t, B, topk)
    assert S * H * (plan.K + 1) * 256 > 200e9 > E.SCRATCH_LIMIT_BYTES
    groups = E._head_groups(plan, H, Hkv, 128, 2)
    assert len(groups) > 1 and all((b - a) % (H // Hkv) == 0 for a, b in groups)
    with torch.no_grad():
        out, lse = E.moba_attn_varlen_with_lse(q, k, v, cu_t, S, B, topk, gqa=True)
    torch.cuda.synchronize()
    rng = np.random.default_rng(3)
    rep = H // Hkv
    rows = sorted(set(rng.integers(0, S, size=6).tolist() + [0, S - 1, 12 * B, 12 * B - 1]))
    for h in (0, 37, H - 1):
        # the selection of this head's rows: the gate stage alone on a one-head view
        qh = q[:, h:h + 1].contiguous()
        kh = k[:, h // rep:h // rep + 1].contiguous()
        vh = v[:, h // rep:h // rep + 1].contiguous()
        sel_h = E.gate_topk(qh, E.chunk_mean(kh, plan), plan)
        for s in rows:
            ref, ref_lse = _row_oracle(qh, kh, vh, sel_h[s, 0].cpu(), s, 0, 0, B, 0)
            err = (out[s, h].float().cpu() - ref).abs().max().item()
            assert err < 2e-2 and err <= 3e-2 * ref.abs().max().item() + 1e-5, (s, h, err)
            assert abs(lse[s, h].item() - ref_lse.item()) < 2e-3
        del qh, kh, vh, sel_h
