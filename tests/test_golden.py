"""Golden vectors under tests/golden/ (written by tests/golden/make_golden.py from the CPU
oracle): the oracle must keep reproducing them, and the HIP operator must match them."""

import glob
import os

import numpy as np
import pytest
import torch

from oracle import moba_oracle as O

FILES = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def load(path):
    z = np.load(path)          # plain arrays only (allow_pickle stays False)
    dtype = torch.float16 if "fp16" in os.path.basename(path) else torch.bfloat16
    t = {k_: torch.from_numpy(z[k_]) for k_ in z.files}
    for name in ("q", "k", "v", "do"):
        t[name] = t[name].view(dtype)
    return t, dtype


def test_fixtures_exist():
    assert len(FILES) >= 2


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
def test_oracle_reproduces_golden(path):
    t, _ = load(path)
    cu = t["cu"].tolist()
    q, k, v = (t[n].clone().requires_grad_(True) for n in ("q", "k", "v"))
    out, lse, sel = O.moba_attn_varlen_oracle(q, k, v, cu, max(b - a for a, b in zip(cu, cu[1:])),
                                              int(t["chunk"]), int(t["topk"]), return_aux=True)
    out.backward(t["do"].float())
    assert torch.equal(sel.to(torch.int32), t["sel"])
    torch.testing.assert_close(out.detach().float(), t["out"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(lse.detach().float(), t["lse"], rtol=1e-5, atol=1e-6)
    for g, name in ((q.grad, "dq"), (k.grad, "dk"), (v.grad, "dv")):
        torch.testing.assert_close(g.float(), t[name], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p) for p in FILES])
def test_operator_matches_golden(path):
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    t, dtype = load(path)
    cu_t = t["cu"].cuda()
    cu = t["cu"].tolist()
    B, topk = int(t["chunk"]), int(t["topk"])
    q, k, v = (t[n].cuda().requires_grad_(True) for n in ("q", "k", "v"))
    out, lse = E.moba_attn_varlen_with_lse(q, k, v, cu_t, max(b - a for a, b in zip(cu, cu[1:])), B, topk)
    out.backward(t["do"].cuda())
    plan = make_plan(cu_t, B, topk)
    sel = E.gate_topk(q.detach(), E.chunk_mean(k.detach(), plan), plan).cpu()
    got = torch.sort(torch.where(sel < 0, torch.full_like(sel, 1 << 30), sel), dim=-1).values
    got = torch.where(got == 1 << 30, torch.full_like(got, -1), got)
    assert torch.equal(got, t["sel"])           # tie-free data: the selection is bit-exact
    # tolerances of the operator tests: max-abs 2e-2, mean-abs 2e-3
    for a, b in ((out, t["out"]), (q.grad, t["dq"]), (k.grad, t["dk"]), (v.grad, t["dv"])):
        err = (a.detach().float().cpu() - b).abs()
        assert err.max() < 2e-2 * max(1.0, b.abs().max().item()) and err.mean() < 2e-3
    assert (lse.cpu() - t["lse"]).abs().max() < 2e-3
