"""Writes tests/golden/small_fp32.npz: seeded inputs of one small fp32 case and what
the CPU oracle (oracle/fm_oracle.py) computes from them, stage by stage.  The
reference holds no golden vectors for this path (its only check draws inputs from
the CUDA generator), so these are the oracle's own outputs, frozen: the CPU test
that recomputes them guards the oracle against drift, the GPU test holds the
library to them.

    python tests/golden/make_fixtures.py

Stages and what the tests compare:
  Y      = A K^T (fp64 sums rounded to fp32)          library: allclose
  lists  = arg-top-Z of Y (value desc, index asc)     library on the stored Y: bit-exact
  qh     = first argmax of A q                         library: bit-exact (margins checked here)
  out, lse of the gathered attention                    library: 1e-4 / 1e-3
  lout, llse of the causal local attention, and the merged (mout, mlse)
  dq, dk, dv of the gathered attention for the stored d_out
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import fm_oracle as O  # noqa: E402

H, G, d, N, C, Z, S, L = 1, 2, 64, 512, 16, 64, 32, 32


def build():
    g = torch.Generator().manual_seed(20240607)
    K = torch.randn(H, N, d, generator=g)
    V = torch.randn(H, N, d, generator=g)
    K[0, 100] = K[0, 7]            # exact ties in every row of Y
    K[0, 300] = K[0, 7]
    K[0, 301] = -K[0, 8]
    K[0, 20] = 0.0                 # a zero row: Y = +0 in every bucket
    Q = torch.randn(H, G * S, d, generator=g)
    A = torch.randn(H, C, d, generator=g)
    A = A / A.norm(dim=-1, keepdim=True)
    KL = torch.randn(H, L, d, generator=g)
    VL = torch.randn(H, L, d, generator=g)
    dO = torch.randn(H, G * S, d, generator=g)
    scale = d ** -0.5
    Y = O.project(A, K)
    lists = O.argtopz(Y, Z)                                      # [H,C,Z]
    sc = O.qhash_scores(A, Q)
    qh = O.argmax_first(sc)
    top2 = sc.topk(2, dim=-1).values
    assert float((top2[..., 0] - top2[..., 1]).min()) > 1e-3, "hash margins too small for a bit-exact fixture"
    cnt = torch.full((H, C), Z)
    out, lse = O.hashed_attention_gather(Q, K, V, lists.reshape(-1), cnt, qh, scale)
    lo, ll = O.local_attention(Q.reshape(1, H * G, S, d), KL.reshape(1, H, L, d), VL.reshape(1, H, L, d), scale, True)
    lo, ll = lo[0].reshape(H, G * S, d), ll[0].reshape(H, G * S)
    mo, ml = O.lse_merge_closed_form(lo.float(), ll, out.float(), lse)
    dq, dk, dv = O.hashed_attention_backward_gather(Q, K, V, lists.reshape(-1), cnt, qh, out, lse, dO, scale)
    t = dict(K=K, V=V, Q=Q, A=A, KL=KL, VL=VL, dO=dO, Y=Y, lists=lists.to(torch.int32), qh=qh.to(torch.int32),
             out=out, lse=lse, lout=lo, llse=ll, mout=mo.float(), mlse=ml.float(), dq=dq.float(), dk=dk.float(),
             dv=dv.float())
    return {k: v.numpy() for k, v in t.items()}


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_fp32.npz")
    np.savez_compressed(path, **build(), dims=np.array([H, G, d, N, C, Z, S, L]))
    print(path, os.path.getsize(path), "bytes")
