"""Writes the golden vectors of this folder: seeded inputs and the outputs, selection and
gradients that the CPU oracle (oracle/moba_oracle.py) gives for them.

The reference holds no stored vectors for this path (its tests are relational, on data drawn on
the device), and it was not imported to make these: they freeze the oracle, whose functions are
pinned independently in tests/test_oracle.py.  Run from the repository root:

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import moba_oracle as O  # noqa: E402

CASES = {
    # name: (cu_seqlens, heads, chunk, topk, dtype, seed)
    "varlen_bf16": ([0, 50, 128], 1, 16, 3, torch.bfloat16, 1),
    "single_fp16": ([0, 96], 2, 16, 4, torch.float16, 2),
}


def build(cu, H, B, topk, dtype, seed):
    S = cu[-1]
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn((S, H, 128), generator=g, dtype=torch.float32).to(dtype) for _ in range(4))
    qc, kc, vc = (x.clone().requires_grad_(True) for x in (q, k, v))
    out, lse, sel = O.moba_attn_varlen_oracle(qc, kc, vc, cu, max(b - a for a, b in zip(cu, cu[1:])), B, topk,
                                              return_aux=True)
    out.backward(do.float())
    bits = lambda x: x.view(torch.int16).numpy()
    return dict(cu=np.asarray(cu, dtype=np.int32), chunk=np.int32(B), topk=np.int32(topk),
                q=bits(q), k=bits(k), v=bits(v), do=bits(do), sel=sel.numpy().astype(np.int32), lse=lse.detach().float().numpy(),
                out=out.detach().float().numpy(), dq=qc.grad.float().numpy(),
                dk=kc.grad.float().numpy(), dv=vc.grad.float().numpy())


if __name__ == "__main__":
    for name, (cu, H, B, topk, dtype, seed) in CASES.items():
        np.savez(os.path.join(HERE, name + ".npz"), **build(cu, H, B, topk, dtype, seed))
        print("wrote", name)
