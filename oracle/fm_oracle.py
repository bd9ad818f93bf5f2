"""CPU oracle for the indexed-memory attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this file:
only the test-suite, the smoke check and the benchmark's CPU-baseline leg use
it, and only as the checker.  Every function restates, in eager torch / numpy
on the CPU, what the reference computes; the citation after each name is the
reference file:line it follows (``tk`` = triton_kernel.py, ``mem`` = memory.py,
``RM`` = README.md under /root/reference).

Conventions (README letters): C buckets, Z keys per bucket, N memory keys,
H KV heads ("batch rows" of the kernel), G query heads per KV head, S query
tokens, d head dimension.  Kernel-side layouts are batch-first:
``A [H,C,d]``, ``K,V [H,N,d]``, ``q [H,S',d]`` with ``S' = G*S``.

How each function is pinned (tests/test_oracle_*.py):
  project            -- torch.matmul in fp64, hand-computed tiny case
  argtopz            -- brute-force O(N^2) rank count on crafted ties, +-0, inf
  qhash              -- brute force first-max scan
  group_queries      -- numpy argsort(kind="stable") / numpy.unique, round trip
  hashed_attention_* -- two independent formulations (per-query gather vs the
                        reference's dense-masked procedure) against each other,
                        C=1,Z=N == full softmax (torch.logsumexp / SDPA),
                        Z=1 == V[idx]; invariants on the LSE
  *_backward_*       -- torch autograd (fp64) through an independent dense
                        softmax over the same visible pairs, alone and as part
                        of a larger softmax (merged out / lse); the two
                        formulations (dense-masked, gather) against each other
  calc_ref_centroids -- brute-force loops over (query, rank) on a tiny input
  update_out_and_lse -- closed form logaddexp / convex combination, split test
  local_attention    -- torch SDPA (math path) + torch.logsumexp.
                        PARITY UNPINNED against the reference: the reference
                        calls attention_forward (mem:302) but ships no
                        definition; only the call-site semantics are followed.
  compute_centroids  -- centroid_topk=1 special case, unit-norm rows,
                        brute-force loop version
  kmeans_spherical   -- objective monotonicity, unit rows, scikit-free brute
                        force on tiny inputs.  The reference has no code for it
                        (RM:37-45 is prose); PARITY UNPINNED against reference
                        code, pinned by the README's definition.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

LN2 = math.log(2.0)
LOG2E = 1.44269504  # the constant the reference kernel multiplies by (tk:195)


# --------------------------------------------------------------------------
# a14  initial centroids                                          mem:489-493
# --------------------------------------------------------------------------
def init_centroids(n_buckets: int, d: int, dtype=torch.float32) -> torch.Tensor:
    """``RandomState(42).randn(C, d)`` cast to the key dtype; not normalised."""
    rng = np.random.RandomState(42)
    return torch.tensor(rng.randn(n_buckets, d), dtype=dtype)


# --------------------------------------------------------------------------
# a1  projection                                      mem:261, tk:277, RM:25
# --------------------------------------------------------------------------
def project(A: torch.Tensor, K: torch.Tensor, out_dtype=torch.float32) -> torch.Tensor:
    """``Y[h,c,n] = sum_d A[h,c,d] * K[h,n,d]`` (tk:277 ``'bzd,bjd->bzj'``).

    Inputs are taken at their stored precision (bf16 values are exact in
    fp32), products are accumulated in fp64 and rounded once to ``out_dtype``.
    """
    Y = torch.einsum('bzd,bjd->bzj', A.double(), K.double())
    return Y.to(out_dtype)


# --------------------------------------------------------------------------
# a2  arg-top-Z                                       mem:273, tk:278, RM:27
# --------------------------------------------------------------------------
def _canon(Y: torch.Tensor) -> torch.Tensor:
    # -0.0 and +0.0 compare equal; adding +0.0 makes the bits agree as well.
    return Y + 0.0


def argtopz(Y: torch.Tensor, Z: int) -> torch.Tensor:
    """Indices of the ``min(Z, N)`` largest entries of every row of ``Y``.

    The reference calls ``torch.topk`` (mem:273, with the ``min`` clamp), whose
    order among equal values is unspecified.  The contract here fixes it:
    value descending, then key index ascending -- i.e. the first ``Z`` entries
    of a *stable* descending sort.  NaN sorts as the largest value.
    """
    N = Y.shape[-1]
    k = min(int(Z), N)
    order = torch.sort(_canon(Y.float()), dim=-1, descending=True, stable=True)[1]
    return order[..., :k].contiguous()


# --------------------------------------------------------------------------
# a3  query hash                                   mem:281-283, tk:280-281, RM:29
# --------------------------------------------------------------------------
def qhash_scores(A: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """fp32 scores ``[H,S',C]`` (tk:280 ``'bzd,bid->biz'``), fp64 accumulate."""
    return torch.einsum('bzd,bid->biz', A.double(), q.double()).float()


def argmax_first(scores: torch.Tensor) -> torch.Tensor:
    """``torch.argmax`` over the last axis; first index wins among equal maxima."""
    return torch.argmax(scores, dim=-1)


def qhash(A: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    return argmax_first(qhash_scores(A, q))


# --------------------------------------------------------------------------
# a16  bucket occupancy                                          mem:285-286
# --------------------------------------------------------------------------
def bin_counts(q_hashes: torch.Tensor, n_buckets: int) -> torch.Tensor:
    H = q_hashes.shape[0]
    flat = q_hashes.reshape(H, -1)
    out = flat.new_zeros((H, n_buckets))
    out.scatter_add_(1, flat, torch.ones_like(flat))
    return out


# --------------------------------------------------------------------------
# a4  window filter + flatten                                    mem:128-142
# --------------------------------------------------------------------------
def window_filter(k_hashes_bcz: torch.Tensor, lo: int, hi: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Keep bucket entries in ``[lo, hi)``; returns (flat re-based indices in
    row-major ``[H,C,*]`` order, per-bucket counts ``[H,C]``)."""
    mask = torch.logical_and(lo <= k_hashes_bcz, k_hashes_bcz < hi)
    counts = mask.to(torch.long).sum(-1)
    flat = k_hashes_bcz[mask] - lo
    return flat, counts


# --------------------------------------------------------------------------
# a5  query grouping                                              tk:75-88
# --------------------------------------------------------------------------
def group_queries(q_hashes: torch.Tensor, n_buckets: int):
    """Host-side grouping the reference does before the kernel launch.

    Returns ``(perm [B,S'], group_bucket, group_count, group_offset)`` where
    ``perm`` is the stable ascending sort permutation per row and groups are
    the distinct (row, bucket) pairs in (row, bucket) order; ``group_offset``
    is the exclusive prefix sum of ``group_count`` over the flattened
    ``B*S'`` sorted query axis (tk:84).
    """
    B, S = q_hashes.shape
    qh = q_hashes.numpy()
    perm = np.argsort(qh, axis=1, kind='stable')
    sorted_h = np.take_along_axis(qh, perm, axis=1)
    flat = (sorted_h + np.arange(B)[:, None] * n_buckets).reshape(-1)
    uniq, counts = np.unique(flat, return_counts=True)  # sorted => consecutive
    offsets = np.concatenate([[0], np.cumsum(counts)[:-1]])
    return (torch.from_numpy(perm), torch.from_numpy(uniq % n_buckets),
            torch.from_numpy(counts), torch.from_numpy(offsets))


def bucket_offsets(k_hash_counts: torch.Tensor) -> torch.Tensor:
    """Exclusive prefix sum over the flattened ``[B,C]`` counts (tk:86-88)."""
    flat = k_hash_counts.reshape(-1)
    cs = torch.cumsum(flat, 0)
    return torch.cat([flat.new_zeros(1), cs[:-1]]).reshape(k_hash_counts.shape)


# --------------------------------------------------------------------------
# a6-a8  bucket-gathered attention, formulation 1: per query, fp64
# --------------------------------------------------------------------------
def _finfo_min(dtype) -> float:
    return torch.finfo(dtype).min


def hashed_attention_gather(q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale,
                            lse_dtype=torch.float32):
    """Definition of the operator (tk:51-119): every query attends to the keys
    listed in the bucket it hashes to.

    q ``[B,S',d]``; k,v ``[B,N,d]``; ``k_hashes`` flat ragged lists in
    row-major (row, bucket) order; ``k_hash_counts [B,C]``; ``q_hashes
    [B,S']``.  Returns ``out [B,S',d]`` in q's dtype and the natural-log LSE
    ``[B,S']`` in ``lse_dtype``.  An empty bucket gives ``out = 0`` and
    ``lse = finfo(lse_dtype).min`` (tk:204-206, 222-223, 114-117).
    """
    B, S, d = q.shape
    C = k_hash_counts.shape[1]
    offs = bucket_offsets(k_hash_counts)
    out = torch.zeros((B, S, d), dtype=torch.float64)
    lse = torch.full((B, S), -math.inf, dtype=torch.float64)
    qd, kd, vd = q.double(), k.double(), v.double()
    for b in range(B):
        for c in range(C):
            sel = (q_hashes[b] == c).nonzero().flatten()
            cnt = int(k_hash_counts[b, c])
            if sel.numel() == 0 or cnt == 0:
                continue
            o0 = int(offs[b, c])
            idx = k_hashes[o0:o0 + cnt].long()
            s = (qd[b, sel] @ kd[b, idx].T) * sm_scale
            l = torch.logsumexp(s, dim=-1)
            out[b, sel] = torch.exp(s - l[:, None]) @ vd[b, idx]
            lse[b, sel] = l
    lse = torch.nan_to_num(lse.to(lse_dtype), nan=0.0,
                           posinf=torch.finfo(lse_dtype).max,
                           neginf=_finfo_min(lse_dtype))
    return out.to(q.dtype), lse


# --------------------------------------------------------------------------
# a6-a8  formulation 2: the reference's dense-masked procedure   tk:327-351
# --------------------------------------------------------------------------
def hashed_attention_dense_masked(q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale,
                                  compute_dtype=torch.float64):
    """Dense scores + scatter mask + softmax, as the reference's own test does
    (tk:327-351; mem:74-103 uses the same construction with a sentinel column
    for masked-out entries).  A fully masked row is reported the way the
    *kernel* defines it (0, finfo.min), not with the dense procedure's
    uniform-average artefact.
    """
    B, S, d = q.shape
    N = k.shape[1]
    C = k_hash_counts.shape[1]
    offs = bucket_offsets(k_hash_counts)
    mask = torch.zeros((B, S, N + 1), dtype=torch.bool)
    zmax = int(k_hash_counts.max()) if k_hash_counts.numel() else 0
    # padded [B,C,zmax] table with sentinel N in unused slots (mem:84)
    table = torch.full((B, C, max(zmax, 1)), N, dtype=torch.long)
    for b in range(B):
        for c in range(C):
            cnt = int(k_hash_counts[b, c])
            o0 = int(offs[b, c])
            table[b, c, :cnt] = k_hashes[o0:o0 + cnt].long()
    b_idx = torch.arange(B)
    k_idx = table[b_idx[:, None], q_hashes.long()]          # B S' zmax
    mask.scatter_(-1, k_idx, True)
    mask = mask[:, :, :-1]
    scores = torch.einsum('bid,bjd->bij', q.to(compute_dtype), k.to(compute_dtype)) * sm_scale
    fmin = torch.finfo(compute_dtype).min
    scores = scores.masked_fill(~mask, fmin)
    smax = scores.max(dim=-1, keepdim=True)[0]
    e = torch.exp(scores - smax)
    e = e.masked_fill(~mask, 0.0)
    esum = e.sum(-1, keepdim=True)
    any_key = mask.any(-1, keepdim=True)
    lse = torch.where(any_key, torch.log(esum) + smax, torch.full_like(smax, -math.inf)).squeeze(-1)
    P = torch.where(any_key, e / esum.clamp(min=1e-300), torch.zeros_like(e))
    out = torch.einsum('bij,bjd->bid', P, v.to(compute_dtype))
    lse32 = torch.nan_to_num(lse.float(), nan=0.0, posinf=torch.finfo(torch.float32).max,
                             neginf=_finfo_min(torch.float32))
    return out.to(q.dtype), lse32


# --------------------------------------------------------------------------
# a6-a8  formulation 3: arithmetic order of the device kernel    tk:137-272
# --------------------------------------------------------------------------
def hashed_attention_blocked(q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale,
                             block_k: int = 128, ref_lse_rounding: bool = False):
    """Follows the reference kernel's rounding points: base-2 online softmax
    with ``sm_scale*1.44269504`` (tk:195), masked lanes at -1e6 (tk:250),
    ``l`` initialised to 1 and ``m`` to -inf (tk:204-205), denominator summed
    in fp32 from unrounded ``p`` while ``p`` is rounded to the input dtype
    before ``P.V`` (tk:253-263), ``o = acc/l`` cast to the input dtype and
    ``lse2 = m + log2(l)`` (tk:222-223); then ``lse = lse2 * ln2`` and
    ``nan_to_num`` (tk:111-117).  With ``ref_lse_rounding`` the LSE is rounded
    to q's dtype before the multiply, as the reference does (tk:111).
    """
    B, S, d = q.shape
    C = k_hash_counts.shape[1]
    offs = bucket_offsets(k_hash_counts)
    out = torch.zeros_like(q)
    lse2 = torch.full((B, S), -math.inf, dtype=torch.float32)
    scale2 = np.float32(sm_scale * LOG2E)
    for b in range(B):
        for c in range(C):
            sel = (q_hashes[b] == c).nonzero().flatten()
            if sel.numel() == 0:
                continue
            cnt = int(k_hash_counts[b, c])
            o0 = int(offs[b, c])
            idx_all = k_hashes[o0:o0 + cnt].long()
            qb = q[b, sel]
            m = torch.full((sel.numel(),), -math.inf, dtype=torch.float32)
            l = torch.ones(sel.numel(), dtype=torch.float32)
            acc = torch.zeros((sel.numel(), d), dtype=torch.float32)
            for j0 in range(0, cnt, block_k):
                idx = idx_all[j0:j0 + block_k]
                s = (qb.float() @ k[b, idx].float().T) * scale2
                m_new = torch.maximum(m, s.max(-1)[0])
                p = torch.exp2(s - m_new[:, None])
                alpha = torch.exp2(m - m_new)
                l = l * alpha + p.sum(-1)
                acc = acc * alpha[:, None] + p.to(q.dtype).float() @ v[b, idx].float()
                m = m_new
            out[b, sel] = (acc / l[:, None]).to(q.dtype)
            lse2[b, sel] = m + torch.log2(l)
    if ref_lse_rounding:
        lse = lse2.to(q.dtype) * LN2
    else:
        lse = lse2 * np.float32(LN2)
    lse = torch.nan_to_num(lse, nan=0.0, posinf=torch.finfo(lse.dtype).max,
                           neginf=_finfo_min(lse.dtype))
    return out, lse


# --------------------------------------------------------------------------
# a15  single-device composite                                    tk:275-286
# --------------------------------------------------------------------------
def attention_hash(q, k, v, centroids, bucket_size, sm_scale, window=None):
    """project -> arg-top-Z -> query hash -> window mask -> gathered attention.
    The reference hard-codes a perf-test window at tk:283; here the window
    defaults to all keys ``[0, N)``."""
    N = k.shape[1]
    Y = project(centroids, k)
    kh = argtopz(Y, bucket_size)
    qh = qhash(centroids, q)
    lo, hi = (0, N) if window is None else window
    flat, counts = window_filter(kh, lo, hi)
    out, lse = hashed_attention_gather(q, k, v, flat + lo, counts, qh, sm_scale)
    return out, lse, kh, qh


# --------------------------------------------------------------------------
# mem:74-103  dense-masked oracle with window sentinel (memory.py layouts)
# --------------------------------------------------------------------------
def ring_attention_masked_forward_ref(k_hashes_zhj, q_hashes_hgi, q, k, v, sm_scale, rank):
    """memory.py layouts: ``k_hashes [C,H,Z]`` global key indices, ``q_hashes
    [H,G,S]``, ``q [1,H*G,S,d]``, ``k,v [1,H,N,d]``; only indices inside
    ``[rank*N,(rank+1)*N)`` take part (mem:83-86)."""
    bs, n_heads, S, d = q.shape
    _, H, N, _ = k.shape
    G = n_heads // H
    h_idx = torch.arange(H)
    mask = torch.zeros((bs, H, G, S, N + 1), dtype=torch.bool)
    k_idx = k_hashes_zhj[q_hashes_hgi, h_idx[:, None, None]]         # H G S Z
    m = torch.logical_and(rank * N <= k_idx, k_idx < (rank + 1) * N)
    k_idx = (k_idx - rank * N) * m + (N * ~m)
    mask.scatter_(-1, k_idx.unsqueeze(0), m.unsqueeze(0))
    mask = mask[..., :-1]
    scores = torch.einsum('bhgid,bhjd->bhgij', q.double().view(bs, H, G, S, d), k.double()) * sm_scale
    scores = scores.masked_fill(~mask, torch.finfo(torch.float64).min)
    smax = scores.max(-1, keepdim=True)[0]
    e = torch.exp(scores - smax)
    esum = e.sum(-1, keepdim=True)
    lse = torch.log(esum) + smax
    P = (e / esum).masked_fill(~mask, 0.0)
    out = torch.einsum('bhgij,bhjd->bhgid', P, v.double())
    return out.reshape(q.shape).to(q.dtype), lse.reshape(q.shape[:-1]).float()


def ring_attention_masked_forward(k_hashes_zhj, q_hashes_hgi, q, k, v, sm_scale, rank,
                                  lse_dtype=torch.float32):
    """mem:106-163 restated on top of the gather formulation."""
    bs, n_heads, S, d = q.shape
    _, H, N, _ = k.shape
    kh = k_hashes_zhj.permute(1, 0, 2)
    flat, counts = window_filter(kh, rank * N, (rank + 1) * N)
    out, lse = hashed_attention_gather(q.reshape(H, -1, d), k.reshape(H, -1, d), v.reshape(H, -1, d),
                                       flat, counts, q_hashes_hgi.reshape(H, -1), sm_scale,
                                       lse_dtype=lse_dtype)
    return out.reshape(bs, n_heads, S, d), lse.reshape(bs, n_heads, S)


# --------------------------------------------------------------------------
# f1  backward of the gathered attention                       mem:166-206
# --------------------------------------------------------------------------
def ring_attention_masked_backward_ref(k_hashes_zhj, q_hashes_hgi, d_out, q, k, v, out, softmax_lse, sm_scale,
                                       rank):
    """mem:166-206 restated in fp64 (dense, masked): with ``P = exp(s - lse)`` on
    the visible (query, key) pairs, ``dV = P^T dO``, ``dP = dO V^T``, ``D =
    rowsum(dO * O)``, ``dS = P * (dP - D)``, ``dQ = scale * dS K``, ``dK =
    scale * dS^T Q``.  ``out`` / ``softmax_lse`` may be those of a larger
    softmax the gathered keys are only a part of (the merged result).  Layouts
    as in :func:`ring_attention_masked_forward_ref`; returns ``(dQ [1,H*G,S,d],
    dK [1,H,N,d], dV [1,H,N,d])`` in fp64."""
    bs, n_heads, S, d = q.shape
    _, H, N, _ = k.shape
    G = n_heads // H
    h_idx = torch.arange(H)
    mask = torch.zeros((bs, H, G, S, N + 1), dtype=torch.bool)
    k_idx = k_hashes_zhj[q_hashes_hgi, h_idx[:, None, None]]         # H G S Z
    m = torch.logical_and(rank * N <= k_idx, k_idx < (rank + 1) * N)
    k_idx = (k_idx - rank * N) * m + (N * ~m)
    mask.scatter_(-1, k_idx.unsqueeze(0), m.unsqueeze(0))
    mask = mask[..., :-1]
    shape = (bs, H, G, S, d)
    qd, dod, od = q.double().view(shape), d_out.double().view(shape), out.double().view(shape)
    kd, vd = k.double(), v.double()
    scores = torch.einsum('bhgid,bhjd->bhgij', qd, kd) * sm_scale
    P = torch.exp(scores - softmax_lse.double().view(bs, H, G, S, 1)).masked_fill(~mask, 0.0)
    dV = torch.einsum('bhgij,bhgid->bhjd', P, dod)
    dP = torch.einsum('bhgid,bhjd->bhgij', dod, vd)
    D = (dod * od).sum(-1, keepdim=True)
    dS = P * (dP - D)
    dQ = torch.einsum('bhgij,bhjd->bhgid', dS, kd) * sm_scale
    dK = torch.einsum('bhgij,bhgid->bhjd', dS, qd) * sm_scale
    return dQ.reshape(bs, n_heads, S, d), dK, dV


def hashed_attention_backward_gather(q, k, v, k_hashes, k_hash_counts, q_hashes, out, lse, d_out, sm_scale):
    """The same gradients on the gather formulation (the layouts of
    :func:`hashed_attention_gather`: ``q,out,d_out [H,Sq,d]``, ``k,v [H,N,d]``,
    flat bucket lists): per query only its bucket's keys are visited.  fp64."""
    H, Sq, d = q.shape
    N = k.shape[1]
    off = bucket_offsets(k_hash_counts)
    dq = torch.zeros((H, Sq, d), dtype=torch.float64)
    dk = torch.zeros((H, N, d), dtype=torch.float64)
    dv = torch.zeros((H, N, d), dtype=torch.float64)
    for h in range(H):
        for i in range(Sq):
            b = int(q_hashes[h, i])
            c = int(k_hash_counts[h, b])
            if c == 0:
                continue
            idx = k_hashes[int(off[h, b]):int(off[h, b]) + c].long()
            kk, vv = k[h, idx].double(), v[h, idx].double()
            qi, doi = q[h, i].double(), d_out[h, i].double()
            p = torch.exp(kk @ qi * sm_scale - float(lse[h, i]))
            dp = vv @ doi
            ds = p * (dp - float((doi * out[h, i].double()).sum()))
            dq[h, i] = sm_scale * (ds @ kk)
            dk[h].index_add_(0, idx, sm_scale * ds[:, None] * qi[None, :])
            dv[h].index_add_(0, idx, p[:, None] * doi[None, :])
    return dq, dk, dv


# --------------------------------------------------------------------------
# a10  LSE merge                                                  mem:54-71
# --------------------------------------------------------------------------
def update_out_and_lse(out: Optional[torch.Tensor], lse: Optional[torch.Tensor],
                       block_out: torch.Tensor, block_lse: torch.Tensor):
    """Statement-for-statement restatement of mem:55-71 (sigmoid/logsigmoid
    form, in place on the running pair)."""
    block_out = block_out.to(torch.float32)
    block_lse = block_lse.unsqueeze(dim=-1)
    if out is None:
        return block_out, block_lse
    lse_d = block_lse - lse
    out -= torch.sigmoid(lse_d) * (out - block_out)
    lse -= torch.nn.functional.logsigmoid(-lse_d)
    return out, lse


def lse_merge_closed_form(out_a, lse_a, out_b, lse_b):
    """What mem:55-71 equals mathematically: ``lse = logaddexp(a, b)`` and the
    softmax-weighted convex combination of the two outputs (fp64)."""
    la, lb = lse_a.double(), lse_b.double()
    l = torch.logaddexp(la, lb)
    wa = torch.exp(la - l)[..., None]
    wb = torch.exp(lb - l)[..., None]
    return wa * out_a.double() + wb * out_b.double(), l


# --------------------------------------------------------------------------
# a11  dense local attention                     call site mem:302-304 only
# --------------------------------------------------------------------------
def local_attention(q, k, v, sm_scale, causal: bool = True):
    """``attention_forward(q, k_self, v_self, sm_scale, True)`` (mem:302): GQA
    softmax attention returning ``(out, lse)``.  ``q [1,H*G,S,d]``, ``k,v
    [1,H,L,d]``.  With ``causal`` query ``i`` sees local keys ``j <= i + (L -
    S)`` (bottom-right aligned; equals the usual lower triangle when
    ``L == S``).  The reference ships no definition of this function, so
    parity with it is unpinned; the textbook definition is what is restated.
    """
    bs, n_heads, S, d = q.shape
    _, H, L, _ = k.shape
    G = n_heads // H
    s = torch.einsum('bhgid,bhjd->bhgij', q.double().view(bs, H, G, S, d), k.double()) * sm_scale
    if causal:
        i = torch.arange(S)[:, None]
        j = torch.arange(L)[None, :]
        s = s.masked_fill(~(j <= i + (L - S)), -math.inf)
    lse = torch.logsumexp(s, dim=-1)
    P = torch.exp(s - lse[..., None])
    P = torch.nan_to_num(P, nan=0.0)
    out = torch.einsum('bhgij,bhjd->bhgid', P, v.double())
    lse32 = torch.nan_to_num(lse.float(), neginf=_finfo_min(torch.float32))
    return out.reshape(bs, n_heads, S, d).to(q.dtype), lse32.reshape(bs, n_heads, S)


# --------------------------------------------------------------------------
# a12  top-k-mean centroids                           mem:209-231, 256-258
# --------------------------------------------------------------------------
def compute_centroids(kq, centroids, n_hashes, n_groups, centroid_topk, normalize=True):
    """``kq [H*G, N, d]``, ``centroids [C,d]`` -> ``A [C,H,d]``.

    mem:214-217 normalise rows (norm clamped at 1e-6); mem:219-221 per
    (centroid, head) the ``centroid_topk`` most similar rows (ties: lower
    index first, the same rule as arg-top-Z); mem:224-229 gather and average
    over the ``G*topk`` rows of a KV head; mem:256-258 (world size 1: the
    all-reduce is the identity) L2-normalise without clamp.
    """
    n_heads, N, d = kq.shape
    H = n_heads // n_groups
    x = kq.double()
    x = x / x.norm(dim=-1, keepdim=True).clamp(min=1e-6)
    x = x.to(kq.dtype).double()          # the reference keeps kq_hash in the input dtype (mem:217)
    scores = torch.einsum('zd,hid->zhi', centroids.double(), x)        # C HG N
    top = argtopz(scores.float(), centroid_topk)                        # C HG k
    h_idx = torch.arange(n_heads)
    picked = x[h_idx[None, :, None], top]                               # C HG k d
    picked = picked.reshape(n_hashes, H, n_groups * top.shape[-1], d)
    A = picked.mean(dim=2)
    if normalize:
        A = A / A.norm(dim=-1, keepdim=True)
    return A.to(kq.dtype)


# --------------------------------------------------------------------------
# a13  spherical K-means                                          RM:37-45
# --------------------------------------------------------------------------
def l2_normalize(X: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    Xd = X.double()
    return (Xd / Xd.norm(dim=-1, keepdim=True).clamp(min=eps)).to(X.dtype)


def kmeans_assign(X: torch.Tensor, cent: torch.Tensor) -> torch.Tensor:
    """Label = first index attaining ``max_c cent[c] . x`` (RM:41)."""
    return torch.argmax((X.double() @ cent.double().T).float(), dim=-1)


def kmeans_update(X: torch.Tensor, labels: torch.Tensor, prev: torch.Tensor) -> torch.Tensor:
    """Mean of the members, re-normalised to unit length (RM:41-43).  A
    cluster without members keeps its previous centroid (the reference has no
    rule; this is the documented one)."""
    C, d = prev.shape
    sums = torch.zeros((C, d), dtype=torch.float64)
    sums.index_add_(0, labels, X.double())
    cnt = torch.bincount(labels, minlength=C)
    new = sums / cnt.clamp(min=1)[:, None]
    nrm = new.norm(dim=-1, keepdim=True)
    new = new / nrm.clamp(min=1e-12)
    keep = (cnt == 0) | (nrm.squeeze(-1) < 1e-12)
    new[keep] = prev.double()[keep]
    return new


def kmeans_spherical(X: torch.Tensor, init: torch.Tensor, iters: int):
    """``X [N,d]`` unit rows, ``init [C,d]`` -> (centroids fp64 ``[C,d]``,
    last labels).  ``iters`` full Lloyd iterations (assign, update)."""
    cent = init.double()
    labels = None
    for _ in range(iters):
        labels = kmeans_assign(X, cent)
        cent = kmeans_update(X, labels, cent)
    return cent, labels



# --------------------------------------------------------------------------
# f2  target of the learned projection                         mem:428-456
# --------------------------------------------------------------------------
def calc_ref_centroids(q_self: torch.Tensor, k: torch.Tensor, topk: int = 128) -> torch.Tensor:
    """mem:428-456 in fp64: scores ``q.k`` per (batch, kv head, group), the
    ``min(topk, N)`` best keys per query (ties: lower key index, the rule of
    :func:`argtopz`; the reference's ``torch.topk`` leaves them open), every
    query scatter-added onto its keys (mem:449-450), divided by ``topk`` and by
    the norm clamped at 1e-6.  Returns ``[B, H, G, N, d]`` fp64."""
    B, n_heads, S, d = q_self.shape
    _, H, N, _ = k.shape
    G = n_heads // H
    _topk = min(topk, N)
    qa = q_self.double().reshape(B, H, G, S, d)
    scores = torch.einsum('bhgid,bhjd->bhgij', qa, k.double())
    best = argtopz(scores.reshape(-1, N), _topk).reshape(B, H, G, S, _topk)
    cent = torch.zeros((B, H, G, N, d), dtype=torch.float64)
    idx = best.reshape(B, H, G, S * _topk, 1).expand(-1, -1, -1, -1, d)
    src = qa.unsqueeze(-2).expand(-1, -1, -1, -1, _topk, -1).reshape(B, H, G, S * _topk, d)
    cent.scatter_add_(3, idx, src)
    cent = cent / _topk
    return cent / cent.norm(p=2, dim=-1, keepdim=True).clamp(min=1e-6)
