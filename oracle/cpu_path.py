"""Eager-PyTorch CPU run of the indexed-memory path, used as the benchmark's
CPU baseline and by the smoke check.

TEST / MEASUREMENT INFRASTRUCTURE ONLY (never imported by the package).  It is
the reference's own sequence of torch calls restated for the CPU:
einsum projection (memory.py:261) -> arg-top-Z (memory.py:273, with the
index-ascending tie rule) -> einsum + argmax hash (memory.py:281-283) ->
per-bucket gathered softmax attention (what triton_kernel.py:137-272 computes)
-> LSE merge with dense local attention (memory.py:302-305, 332).  Arithmetic
is fp32 on the stored (possibly bf16) values.
"""
from __future__ import annotations

import math
import time
from typing import Optional, Tuple

import torch


def build_rows(A_rows: torch.Tensor, K: torch.Tensor, Z: int) -> torch.Tensor:
    """Bucket lists for some rows of A against all keys of one head:
    ``A_rows [R,d]``, ``K [N,d]`` -> ``[R, min(Z,N)]`` int64."""
    Y = A_rows.float() @ K.float().T
    order = torch.sort(Y + 0.0, dim=-1, descending=True, stable=True)[1]
    return order[:, :min(Z, K.shape[0])]


def hash_queries(A: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """``A [C,d]``, ``q [n,d]`` -> bucket ids ``[n]``."""
    return torch.argmax(q.float() @ A.float().T, dim=-1)


def bucket_attention(q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, idx: torch.Tensor,
                     sm_scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Queries ``q [n,d]`` that share one bucket ``idx [Z]`` -> (out fp32 [n,d], lse [n])."""
    Kb, Vb = K[idx].float(), V[idx].float()
    s = (q.float() @ Kb.T) * sm_scale
    lse = torch.logsumexp(s, dim=-1)
    return torch.exp(s - lse[:, None]) @ Vb, lse


def hashed_attention(q, K, V, A, lists, sm_scale):
    """One head: ``q [n,d]``, ``lists [C,Z]`` -> (out fp32 [n,d], lse [n], hashes)."""
    h = hash_queries(A, q)
    out = torch.zeros(q.shape, dtype=torch.float32)
    lse = torch.full((q.shape[0],), torch.finfo(torch.float32).min)
    for c in torch.unique(h).tolist():
        sel = (h == c).nonzero().flatten()
        o, l = bucket_attention(q[sel], K, V, lists[c], sm_scale)
        out[sel], lse[sel] = o, l
    return out, lse, h


def local_attention(q, k, v, sm_scale, q_pos=None, n_tokens=None):
    """Queries ``q [n,d]`` at token positions ``q_pos [n]`` of a sequence of
    ``n_tokens`` against local keys ``k,v [L,d]`` -> (out fp32, lse).  Causal,
    bottom-right aligned: position i sees keys j <= i + (L - n_tokens); no
    mask when ``q_pos`` is None."""
    s = (q.float() @ k.float().T) * sm_scale
    if q_pos is not None:
        L = k.shape[0]
        j = torch.arange(L)[None, :]
        s = s.masked_fill(j > q_pos[:, None] + (L - n_tokens), -math.inf)
    lse = torch.logsumexp(s, dim=-1)
    return torch.exp(s - lse[:, None]) @ v.float(), lse


def merge(out_a, lse_a, out_b, lse_b):
    """memory.py:55-71 in its sigmoid / logsigmoid form."""
    d = lse_b - lse_a
    out = out_a - torch.sigmoid(d)[:, None] * (out_a - out_b)
    lse = lse_a - torch.nn.functional.logsigmoid(-d)
    return out, lse


def time_query_path(q, K, V, A, lists, sm_scale, k_local=None, v_local=None, q_pos=None,
                    n_tokens=None, reps: int = 1) -> float:
    """Seconds per pass of hash + bucket attention (+ local attention + merge)
    for the given queries of one head."""
    best = math.inf
    for _ in range(reps):
        t0 = time.perf_counter()
        out, lse, _ = hashed_attention(q, K, V, A, lists, sm_scale)
        if k_local is not None:
            lo, ll = local_attention(q, k_local, v_local, sm_scale, q_pos, n_tokens)
            merge(lo, ll, out, lse)
        best = min(best, time.perf_counter() - t0)
    return best
