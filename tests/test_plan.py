"""Host-side chunk metadata (moba_amd/plan.py) against the oracle's calc_chunks and
closed forms; runs without a GPU."""

import numpy as np
import pytest

from oracle import moba_oracle as O
from moba_amd.plan import make_plan, FWD_TILE_ROWS, TILE_ROWS


def rand_cu(rng, nseq, lo, hi):
    return np.concatenate([[0], np.cumsum(rng.integers(lo, hi, size=nseq))]).tolist()


@pytest.mark.parametrize("seed", range(20))
def test_plan_tables_match_oracle(seed):
    rng = np.random.default_rng(seed)
    cu = rand_cu(rng, int(rng.integers(1, 6)), 1, 400)
    B = int(rng.integers(1, 80))
    topk = int(rng.integers(1, 6))
    plan = make_plan(cu, B, topk)
    m = O.calc_chunks(cu, B)
    k = O.effective_topk(topk, m["num_filtered_chunk"])
    assert plan.k_eff == k and plan.fallback == (k <= 0)
    if plan.fallback:
        assert plan.host["chunk_tok"].tolist() == cu
        assert plan.N == len(cu) - 1 and plan.K == 0
        return
    assert plan.N == len(m["cu_chunk"]) - 1 and plan.F == m["num_filtered_chunk"]
    assert plan.host["chunk_tok"].tolist() == m["cu_chunk"].tolist()
    assert plan.host["fchunk_tok"].tolist() == m["cu_chunk"][m["filtered_chunk_indices"]].tolist()
    assert plan.host["seq_fbase"][:-1].tolist() == m["first_filtered"].tolist()
    assert plan.K == min(k, int(m["n_chunks"].max()) - 1)
    assert plan.pairs_per_head == O.expected_pair_count(cu, B, k, 1)
    assert plan.P == int(sum(n * (n - 1) // 2 for n in m["n_chunks"]))
    assert plan.flops_per_head * 128 == pytest.approx(O.attention_flops(cu, B, topk, 1, 128))
    lens = np.diff(m["cu_chunk"])
    assert plan.self_tiles == plan.kv_tiles == int(((lens + TILE_ROWS - 1) // TILE_ROWS).sum())
    # every per-head self tile names its chunk: prefix[c] <= t < prefix[c+1]
    stc, pre = plan.host["self_tile_chunk"], plan.host["self_tile_prefix"]
    assert stc.size == plan.self_tiles
    assert all(pre[c] <= t < pre[c + 1] for t, c in enumerate(stc.tolist()))
    # the same for the forward kernel's taller tiles
    assert (TILE_ROWS, FWD_TILE_ROWS) == (128, 256)
    assert plan.fwd_self_tiles == int(((lens + FWD_TILE_ROWS - 1) // FWD_TILE_ROWS).sum())
    stc, pre = plan.host["fwd_self_tile_chunk"], plan.host["fwd_self_tile_prefix"]
    assert stc.size == plan.fwd_self_tiles
    assert all(pre[c] <= t < pre[c + 1] for t, c in enumerate(stc.tolist()))


def brute_force_dense(cu, B, K, d):
    """Token-by-token restatement of the dense-prefix decomposition: attention chunk of every token, number of
    list entries, and for every chunk where the causal rows of its keys end."""
    achunk_starts, entries, self_end = [], 0, []
    for a, b in zip(cu[:-1], cu[1:]):
        n = -(-(b - a) // B)
        prefix_end = min(b, a + (d + 1) * B)
        achunk_starts.append(a)
        for c in range(n):
            lo, hi = a + c * B, min(b, a + (c + 1) * B)
            if c > d:
                achunk_starts.append(lo)
                entries += (hi - lo) * min(K, c)
                self_end.append(hi)
            else:
                self_end.append(prefix_end)
    return achunk_starts + [cu[-1]], entries, self_end


@pytest.mark.parametrize("seed", range(20))
def test_dense_prefix_tables(seed):
    """The plan with dense prefixes: chunks 0..K of every sequence form one attention chunk, their tokens have no
    list entries, everything about the gate's chunks stays as it is."""
    rng = np.random.default_rng(500 + seed)
    cu = rand_cu(rng, int(rng.integers(1, 6)), 1, 600)
    B = int(rng.integers(1, 80))
    topk = int(rng.integers(2, 7))
    plan = make_plan(cu, B, topk)
    if plan.fallback:
        assert plan.with_dense_prefix() is plan
        return
    assert plan.dense_local == 0 and plan.NA == plan.N and plan.kv_tiles == plan.self_tiles
    assert np.array_equal(plan.host["achunk_tok"], plan.host["chunk_tok"])
    assert np.array_equal(plan.host["chunk_self_end"], plan.host["chunk_tok"][1:])
    assert np.array_equal(plan.host["kv_tile_prefix"], plan.host["self_tile_prefix"])
    dense = plan.with_dense_prefix()
    assert dense.dense_local == plan.K and dense.with_dense_prefix() is dense and plan.with_dense_prefix() is dense
    for name in ("chunk_tok", "seq_fbase", "fchunk_tok", "chunk_fb", "chunk_local", "pair_off", "chunk_fid",
                 "kv_tile_prefix", "kv_tile_chunk", "cu_seqlens"):
        assert np.array_equal(dense.host[name], plan.host[name]), name
    assert (dense.N, dense.F, dense.K, dense.P, dense.cmax, dense.kv_tiles) == \
        (plan.N, plan.F, plan.K, plan.P, plan.cmax, plan.kv_tiles)
    assert dense.flops_per_head == plan.flops_per_head
    achunk, entries, self_end = brute_force_dense(cu, B, plan.K, plan.K)
    assert dense.host["achunk_tok"].tolist() == achunk and dense.NA == len(achunk) - 1
    assert dense.pairs_per_head == entries
    assert dense.host["chunk_self_end"].tolist() == self_end
    # the first attention chunk of every sequence has no history slots; the merge walks the tokens behind it
    for pl, d in ((plan, 0), (dense, plan.K)):
        first_end = [min(b_, a_ + (d + 1) * B) for a_, b_ in zip(cu[:-1], cu[1:])]
        assert pl.host["mrg_start"].tolist() == first_end
        assert np.array_equal(np.diff(pl.host["mrg_prefix"]), np.asarray(cu[1:]) - np.asarray(first_end))
        assert pl.merge_tokens == int(pl.host["mrg_prefix"][-1]) and pl.host["mrg_prefix"][0] == 0
        starts = set(cu[:-1])
        assert pl.host["achunk_direct"].tolist() == [int(t in starts) for t in pl.host["achunk_tok"][:-1].tolist()]
    alen = np.diff(dense.host["achunk_tok"])
    for rows, pre, chunk, count in ((TILE_ROWS, "self_tile_prefix", "self_tile_chunk", dense.self_tiles),
                                    (FWD_TILE_ROWS, "fwd_self_tile_prefix", "fwd_self_tile_chunk", dense.fwd_self_tiles)):
        assert count == int(((alen + rows - 1) // rows).sum()) == dense.host[chunk].size
        assert np.array_equal(np.diff(dense.host[pre]), (alen + rows - 1) // rows)
        assert all(dense.host[pre][c] <= t < dense.host[pre][c + 1] for t, c in enumerate(dense.host[chunk].tolist()))


def test_plan_headline_config_sizes():
    plan = make_plan([0, 131072], 4096, 12)
    assert (plan.N, plan.F, plan.K, plan.P) == (32, 31, 11, 496)
    assert plan.pairs_per_head * 32 == 37486592
    assert plan.flops_per_head * 128 * 32 == pytest.approx(8.301e13, rel=1e-3)
    dense = plan.with_dense_prefix()
    assert (dense.NA, dense.dense_local) == (21, 11) and dense.host["achunk_tok"][:3].tolist() == [0, 49152, 53248]
    assert dense.pairs_per_head == 20 * 4096 * 11 and dense.fwd_self_tiles == plan.fwd_self_tiles


def test_plan_rejects_bad_input():
    with pytest.raises(ValueError):
        make_plan([0, 5, 5, 9], 4, 3)
    with pytest.raises(ValueError):
        make_plan([1, 5], 4, 3)


def test_plan_cache_follows_the_tensor_contents():
    import torch
    cu = torch.tensor([0, 100, 260], dtype=torch.int32)
    a = make_plan(cu, 32, 3)
    assert make_plan(cu, 32, 3) is a                      # same tensor, same version
    assert make_plan(cu.clone(), 32, 3) is a              # equal lengths share one plan
    assert make_plan([0, 100, 260], 32, 3) is a
    cu[1] = 120                                           # in-place update: the version changes
    b = make_plan(cu, 32, 3)
    assert b is not a and b.cu == [0, 120, 260] and a.cu == [0, 100, 260]
    assert b.host["cu_seqlens"].tolist() == [0, 120, 260]
    # a host copy supplied by the caller is used instead of reading the tensor
    c = make_plan(torch.tensor([0, 7, 9], dtype=torch.int32), 4, 2, host_lengths=[0, 7, 9])
    assert c.cu == [0, 7, 9]
    # different chunk size or top-k: different plan
    assert make_plan(cu, 16, 3) is not b and make_plan(cu, 32, 2) is not b


def test_plan_accepts_inference_tensors():
    """A cu_seqlens made under torch.inference_mode() has no version counter: it is planned by value on
    every call (never remembered by identity), so an in-place update inside that mode is seen too."""
    import torch
    with torch.inference_mode():
        cu = torch.tensor([0, 100, 260], dtype=torch.int32)
        assert cu.is_inference()
        a = make_plan(cu, 32, 3)
        assert a.cu == [0, 100, 260] and make_plan(cu, 32, 3) is a
        cu[1] = 120
        assert make_plan(cu, 32, 3).cu == [0, 120, 260]
        assert make_plan(cu, 32, 3, host_lengths=[0, 120, 260]).cu == [0, 120, 260]
    assert make_plan(cu, 32, 3).cu == [0, 120, 260]      # and outside the mode as well


@pytest.mark.parametrize("seed", range(30))
def test_c_planner_equals_python_planner(seed):
    """moba_plan / moba_plan_fill / moba_plan_sizes (host functions of the C ABI, for hosts that are not Python)
    against the numpy planner: same counts, same tables, same buffer sizes."""
    import ctypes
    from moba_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(1000 + seed)
    cu = rand_cu(rng, int(rng.integers(1, 7)), 1, 900)
    B = int(rng.integers(1, 300))
    topk = int(rng.integers(1, 7))
    if seed == 0:
        cu, B, topk = [0, 131072], 4096, 12
    plan = make_plan(cu, B, topk)
    dense = seed % 2
    if dense:
        plan = plan.with_dense_prefix()
    cu_arr = (ctypes.c_int32 * len(cu))(*cu)
    ps, ps2 = _lib.PlanStruct(), _lib.PlanStruct()
    assert lib.moba_plan(cu_arr, len(cu) - 1, B, topk, dense, ctypes.byref(ps)) == 0
    tab = (ctypes.c_int32 * max(1, ps.table_ints))()
    assert lib.moba_plan_fill(cu_arr, len(cu) - 1, B, topk, dense, ctypes.byref(ps2), tab) == 0
    assert bytes(ps) == bytes(ps2)
    tab = np.frombuffer(tab, dtype=np.int32)
    assert (ps.S, ps.nseq, ps.N, ps.F, ps.K, ps.P, ps.cmax, bool(ps.fallback)) == \
        (plan.S, plan.nseq, plan.N, plan.F, plan.K, plan.P, plan.cmax, plan.fallback)
    assert (ps.pairs_per_head, ps.fwd_self_tiles, ps.bwd_self_tiles) == (plan.pairs_per_head, plan.fwd_self_tiles, plan.self_tiles)
    assert (ps.dense_local, ps.NA, ps.kv_tiles) == (plan.dense_local, plan.NA, plan.kv_tiles)
    assert (ps.fwd_tile_rows, ps.bwd_tile_rows) == (FWD_TILE_ROWS, TILE_ROWS)
    assert ps.flops_per_head_per_dim == plan.flops_per_head
    seen = 0
    for name, arr in plan.host.items():
        off = getattr(ps, "off_" + name)
        assert off >= 0 and np.array_equal(tab[off:off + arr.size], arr.astype(np.int32)), name
        seen += arr.size
    assert seen == ps.table_ints
    if plan.fallback:
        assert ps.off_fchunk_tok == ps.off_pair_off == ps.off_chunk_fid == -1
    H, Hkv = 6, 3
    sz = _lib.SizesStruct()
    assert lib.moba_plan_sizes(ctypes.byref(ps), H, Hkv, 128, ctypes.byref(sz)) == 0
    assert sz.fwd_hist_bound == plan.hist_tile_bound(H, FWD_TILE_ROWS) and sz.bwd_hist_bound == plan.hist_tile_bound(H, TILE_ROWS)
    assert sz.sel_ints == plan.S * H * plan.K and sz.cnt_ints == plan.P * H + 1 and sz.seg_off_ints == plan.F * H + 1
    assert sz.seg_dest_ints == max(1, plan.pairs_per_head * H) and sz.part_rows == plan.S * H * (plan.K + 1)
    assert sz.redo_ints == 1 + sz.fwd_hist_bound + plan.fwd_self_tiles * H and sz.kbar_elems == plan.F * Hkv * 128
    assert sz.chunk_mean_workspace_bytes == (lib.moba_chunk_mean_workspace_bytes(Hkv, 128, plan.F, B) if plan.F else 0)


def test_c_planner_rejects_bad_input():
    import ctypes
    from moba_amd import _lib
    lib = _lib.load()
    ps = _lib.PlanStruct()
    for cu in ([0, 5, 5, 9], [1, 5], [0, 4, 3]):
        arr = (ctypes.c_int32 * len(cu))(*cu)
        assert lib.moba_plan(arr, len(cu) - 1, 4, 3, 0, ctypes.byref(ps)) == -1
    arr = (ctypes.c_int32 * 2)(0, 8)
    assert lib.moba_plan(arr, 1, 0, 3, 0, ctypes.byref(ps)) == -1 and lib.moba_plan(arr, 1, 4, 0, 1, ctypes.byref(ps)) == -1
