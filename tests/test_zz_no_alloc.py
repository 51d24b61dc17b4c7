"""moba_chunk_mean_static, the entry point that allocates nothing (its partial sums live in a fixed array
inside the library), against moba_chunk_mean: bit for bit the same chunk means, on calls in a row that share
the array, the later ones with smaller inputs, and a clear error beyond the array's capacity."""

import pytest
import torch

from conftest import make_case

pytestmark = pytest.mark.gpu


def _both(k, cu, B):
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    lib = _lib.load()
    plan = make_plan(torch.tensor(cu, dtype=torch.int32, device="cuda"), B, 3)
    S, H, D = k.shape
    want = E.chunk_mean(k, plan)                      # moba_chunk_mean with a torch-allocated workspace
    got = torch.zeros_like(want)
    rc = lib.moba_chunk_mean_static(E._ptr(k), E._ptr(plan.tables["fchunk_tok"]), E._ptr(got), S, H, D, plan.F, B,
                                    E._strides(None, k), E._dtype_code(k), E._stream(k.device))
    _lib.check(rc, "moba_chunk_mean_static")
    torch.cuda.synchronize()
    return got, want


def test_static_chunk_mean_equals_chunk_mean_on_successive_calls():
    # a large input first (31 chunks x 64 splits x 8 heads: its partial sums take 15.5 MiB of the array) ...
    g = torch.Generator(device="cuda").manual_seed(4)
    k1 = torch.randn((32 * 4096, 8, 128), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    got, want = _both(k1, [0, 32 * 4096], 4096)
    assert want.shape == (31, 8, 128) and torch.equal(got, want)
    # ... then smaller ones, which reuse the front of the array while the rest still holds the old sums
    _, k2, _, _, cu2, _ = make_case(3, 3000, 3, seed=1)
    got, want = _both(k2.cuda(), cu2, 100)
    assert torch.equal(got, want)
    _, k3, _, _, cu3, _ = make_case(1, 1024, 2, seed=2, dtype=torch.float16)
    got, want = _both(k3.cuda(), cu3, 128)
    assert torch.equal(got, want)
    # a strided key tensor ([heads, tokens, dim] seen token-first), as the other entry point reads it in place
    k4 = k2.cuda().transpose(0, 1).contiguous().transpose(0, 1)
    got, want = _both(k4, cu2, 100)
    assert torch.equal(got, want)
    # and the large one again
    got, want = _both(k1, [0, 32 * 4096], 4096)
    assert torch.equal(got, want)


def test_static_chunk_mean_narrows_its_split_to_fit_and_refuses_what_cannot_fit():
    from moba_amd import _lib
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan
    lib = _lib.load()
    cap = lib.moba_chunk_mean_static_capacity()
    assert cap == 32 << 20
    # 64 heads x 47 chunks of 2048: moba_chunk_mean uses 16 token splits there (47 MiB of partial sums), so the
    # static call must take 8 (23.5 MiB) -- with the same result, the sums being exact
    g = torch.Generator(device="cuda").manual_seed(5)
    k = torch.randn((48 * 2048, 64, 128), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    assert lib.moba_chunk_mean_workspace_bytes(64, 128, 47, 2048) == 47 << 20 > cap
    got, want = _both(k, [0, 48 * 2048], 2048)
    assert torch.equal(got, want)
    del k, got, want
    # F * H * 1 KiB beyond the array: refused, nothing launched
    B, F, H = 8, 40000, 1
    S = B * (F + 1)
    k = torch.zeros((S, H, 128), dtype=torch.bfloat16, device="cuda")
    plan = make_plan([0, S], B, 3, device="cuda")
    kbar = torch.full((F, H, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    rc = lib.moba_chunk_mean_static(E._ptr(k), E._ptr(plan.tables["fchunk_tok"]), E._ptr(kbar), S, H, 128, F, B, None,
                                    E._dtype_code(k), E._stream(k.device))
    assert rc == -4 and b"limit" in lib.moba_strerror(rc)
    torch.cuda.synchronize()
    assert bool((kbar == 7.0).all())
