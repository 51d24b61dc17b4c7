"""The operator inside a HIP graph: after one eager call (which reads cu_seqlens once and
caches the plan) a forward launches kernels only, so it can be captured and replayed.  Every
replay is checked against the eager result, with eager work and synchronisations between."""

import pytest
import torch

from conftest import make_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [(2, 4096, 4, 256, 3), (1, 2048, 2, 128, 1)])
def test_forward_graph_replay(batch, seqlen, heads, B, topk):
    from moba_amd import moba_attn_varlen
    q, k, v, _, cu, mx = make_case(batch, seqlen, heads, seed=9)
    q, k, v = q.cuda(), k.cuda(), v.cuda()
    cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
    eager = moba_attn_varlen(q, k, v, cu_t, mx, B, topk)
    torch.cuda.synchronize()

    static_q = q.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up on the capture stream's side
        moba_attn_varlen(static_q, k, v, cu_t, mx, B, topk)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = moba_attn_varlen(static_q, k, v, cu_t, mx, B, topk)
    for it in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_out, eager), it
        # eager work between the replays, on other data
        other = moba_attn_varlen(k, q, v, cu_t, mx, B, topk)
        torch.cuda.synchronize()
        assert torch.isfinite(other.float()).all()
    # new contents in the static input: the replay must follow them
    static_q.copy_(k)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(static_out, moba_attn_varlen(k, k, v, cu_t, mx, B, topk))
