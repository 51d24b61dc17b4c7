"""The operator inside a HIP graph: after one eager call (which reads cu_seqlens once and
caches the plan) a forward launches kernels only, so it can be captured and replayed.  Every
replay is checked against the eager result, with eager work and synchronisations between."""

import pytest
import torch

from conftest import make_case

pytestmark = pytest.mark.gpu


# the third shape has enough tiles for the forward kernel's resident-workgroup form, whose tile counters
# are zeroed by a kernel of the call (so that a replay starts from zero as well)
@pytest.mark.parametrize("batch,seqlen,heads,B,topk", [(2, 4096, 4, 256, 3), (1, 2048, 2, 128, 1), (2, 65536, 8, 1024, 4)])
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


def test_two_streams_at_once():
    """Forward and backward of two problems issued on two streams without waiting in between.  The
    attention kernels keep their workgroups resident and draw tiles from counters: each call has its own
    counters, and with two kernels competing for the CUs not every workgroup is resident from the start --
    the results must be those of the calls made one after the other."""
    from moba_amd import moba_attn_varlen
    cases = []
    for seed, (seqlen, heads, B, topk) in enumerate([(65536, 8, 1024, 4), (49152, 8, 512, 6)]):
        q, k, v, do, cu, mx = make_case(2, seqlen, heads, seed=30 + seed)
        cu_t = torch.tensor(cu, dtype=torch.int32, device="cuda")
        cases.append(([x.cuda() for x in (q, k, v)], do.cuda(), cu_t, mx, B, topk))

    def run(case, stream=None):
        (q, k, v), do, cu_t, mx, B, topk = case
        q, k, v = (x.clone().requires_grad_(True) for x in (q, k, v))
        out = moba_attn_varlen(q, k, v, cu_t, mx, B, topk)
        out.backward(do)
        return out.detach(), q.grad, k.grad, v.grad

    want = [run(c) for c in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(2):
        got = []
        for c, st in zip(cases, streams):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                got.append(run(c))
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            for a, b_ in zip(g, w):
                assert torch.equal(a, b_)
