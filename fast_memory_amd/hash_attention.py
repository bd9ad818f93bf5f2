"""Operator-level API with the reference's names and argument order
(triton_kernel.py): ``attention_hash_varlen`` and ``attention_hash``.

The grouping of queries (sort / unique / cumsum in the reference, with host
synchronisations), the kernel and the un-permute run inside libfastmem; nothing
here reads a value back from the device.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops


def _as_i32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.int32 else t.to(torch.int32)


def attention_hash_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          k_hashes: torch.Tensor, k_hash_counts: torch.Tensor,
                          q_hashes: torch.Tensor, sm_scale: float,
                          lse_dtype: Optional[torch.dtype] = torch.float32) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for ``attention_hash_varlen`` (triton_kernel.py:51-119).

    :param q: ``[batch_size, q_seq_len, d_head]``
    :param k: ``[batch_size, kv_seq_len, d_head]``
    :param v: ``[batch_size, kv_seq_len, d_head]``
    :param k_hashes: flat key indices of all buckets, row-major ``(batch, bucket)``
    :param k_hash_counts: ``[batch_size, C]`` keys per bucket
    :param q_hashes: ``[batch_size, q_seq_len]`` bucket of every query
    :param sm_scale: softmax scale
    :param lse_dtype: ``torch.float32`` (default) returns the fp32 natural-log
        LSE; ``None`` follows the reference's rounding order
        (triton_kernel.py:111-117): the base-2 LSE is rounded to q's dtype and
        multiplied by ln 2 in that dtype (the base-2 value is recovered from
        the fp32 natural-log one, i.e. to one fp32 rounding).
    :return: ``(out [batch, q_seq_len, d_head], lse [batch, q_seq_len])``;
        a query whose bucket holds no key gets ``out = 0`` and
        ``lse = finfo(lse.dtype).min``.
    """
    batch_size, q_seq_len, d_head = q.shape
    _, kv_seq_len, _ = k.shape
    _, n_buckets = k_hash_counts.shape

    assert k.shape[0] == batch_size
    assert k_hash_counts.shape[0] == batch_size
    assert q_hashes.shape[0] == batch_size
    assert q_hashes.shape[1] == q_seq_len, f'{q_hashes.shape} != {q_seq_len}'
    assert d_head == k.shape[-1] == v.shape[-1]
    assert q.is_contiguous()
    assert k.is_contiguous()
    assert v.is_contiguous()
    assert k.stride() == v.stride()

    out, lse = ops.attention_hash_varlen_i32(q, k, v, _as_i32(k_hashes).contiguous(),
                                             _as_i32(k_hash_counts).contiguous(),
                                             _as_i32(q_hashes).contiguous(), sm_scale)
    if lse_dtype is None:
        # the reference's order (triton_kernel.py:111-117): the kernel's base-2 value is rounded to q's
        # dtype first, the product with ln 2 is then formed in that dtype, then nan_to_num
        empty = lse < -1e30
        lse2 = (lse * 1.4426950408889634).to(q.dtype)
        lse = lse2 * 0.6931471805599453
        lse = lse.masked_fill(empty, torch.finfo(lse.dtype).min)
        lse = torch.nan_to_num(lse, nan=0.0, posinf=torch.finfo(lse.dtype).max,
                               neginf=torch.finfo(lse.dtype).min)
    elif lse_dtype != torch.float32:
        lse = torch.nan_to_num(lse.to(lse_dtype), neginf=torch.finfo(lse_dtype).min)
    return out, lse


def sorts_lists(n_queries: int, n_buckets: int) -> bool:
    """Whether :func:`attention_hash`, whose lists serve one call, reorders them by key for the attention:
    from one query per bucket on average up to 96.  The reordering costs 2-5 % of such an attention and
    makes it 25 % faster at 16 queries per bucket, 13 % at 32, 3 % at 64; from about 100 queries per bucket
    the attention is bound by its arithmetic and gains nothing (measured on the reference's harness extents,
    triton_kernel.py:507-528, 65536 keys, 1024 buckets of 3072)."""
    return n_buckets <= n_queries < 96 * n_buckets


def attention_hash(q, k, v, centroids, bucket_size, sm_scale, window=None, key_order=None):
    """Drop-in for the single-device composite ``attention_hash``
    (triton_kernel.py:275-286): project, arg-top-Z, hash, attend.

    ``centroids [batch, C, d]``.  The reference hard-codes a benchmark window
    of key indices at triton_kernel.py:283; ``window=(lo, hi)`` gives the same
    filter, default all keys.  ``key_order``: hand the lists to the attention in
    ascending key order (:func:`ops.lists_key_order`; the same result up to fp32
    rounding, faster row gathers); ``None`` decides by :func:`sorts_lists`."""
    k_hashes = ops.build_index(centroids, k, bucket_size)
    q_hashes = ops.qhash(centroids, q)
    if window is None:
        B, C, Z = k_hashes.shape
        counts = torch.full((B, C), Z, dtype=torch.int32, device=q.device)
        flat = k_hashes.reshape(-1)
        if key_order is None:
            key_order = sorts_lists(q.shape[1], C)
        if key_order:
            off = torch.arange(B * C, dtype=torch.int64, device=q.device) * Z
            flat = ops.lists_key_order(flat, off, counts.reshape(-1), k.shape[1])
    else:
        lo, hi = window
        flat, counts, _ = ops.window_filter(k_hashes, lo, hi)
        flat = flat + lo if lo else flat
    return ops.attention_hash_varlen_i32(q, k, v, flat, counts, q_hashes, sm_scale)


def attention_hash_varlen_backward(d_out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                   out: torch.Tensor, lse: torch.Tensor, k_hashes: torch.Tensor,
                                   k_hash_counts: torch.Tensor, q_hashes: torch.Tensor, sm_scale: float,
                                   staged: Optional[bool] = None, inverse_index=None,
                                   d_lse: Optional[torch.Tensor] = None
                                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gradients of :func:`attention_hash_varlen` w.r.t. ``q``, ``k`` and ``v``.

    The reference registers no gradient for its operator (triton_kernel.py:44-48) and falls back to a
    dense ``[S, N]`` evaluation (memory.py:166-206); this visits only each query's bucket.  ``out`` and
    ``lse`` are the forward's results (fp32 natural-log LSE) or the ones merged with further keys, in
    which case the gradients are the gathered keys' share.

    :param staged: ``True`` takes the path without atomics (bf16 / fp16, d=128: per-bucket bf16 partial rows, then a
        sum per key; needs the inverse of the lists), ``False`` the atomic adds; ``None`` picks the staged
        path when there are at least as many queries per row as buckets, i.e. when most buckets receive
        queries.
    :param d_lse: gradient w.r.t. the returned (natural-log, fp32) LSE ``[batch, q_seq_len]``, for callers that
        differentiate through a merge of partial results done outside; ``None`` = zero.
    :param inverse_index: ``ops.inverse_index(...)`` of these lists, if the caller keeps one (it depends on
        the lists only); built here otherwise.
    :return: ``(dq [batch, q_seq_len, d_head], dk, dv [batch, kv_seq_len, d_head])``; ``dq`` in q's dtype,
        ``dk`` / ``dv`` in fp32 (sums over every bucket a key belongs to).
    """
    batch_size, q_seq_len, d_head = q.shape
    assert d_out.shape == q.shape and out.shape == q.shape and lse.shape == (batch_size, q_seq_len)
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    n_buckets = k_hash_counts.shape[1]
    counts = _as_i32(k_hash_counts).contiguous()
    hashes = _as_i32(q_hashes).contiguous()
    off = ops.bucket_offsets(counts)
    groups = ops.group_queries(hashes, n_buckets)
    lists = _as_i32(k_hashes).contiguous()
    can_stage = q.dtype in (torch.bfloat16, torch.float16) and d_head in (64, 128) and lists.numel() > 0
    auto = staged is None
    if auto:
        staged = can_stage and q_seq_len >= n_buckets and not ops.generic_kernels_forced()
    if staged:
        assert can_stage, "the staged backward takes bf16 or fp16 with d_head = 64 or 128"
        try:
            inv = inverse_index if inverse_index is not None else ops.inverse_index(lists, off, counts, k.shape[1])
            if inv.row_pos[-1] > 0:        # no listed entry at all: nothing to stage, the other form handles it
                return ops.hash_attn_bwd_staged(q, k, v, lists, off, counts, groups, inv, out.contiguous(),
                                                lse.float().contiguous(), d_out.contiguous(), sm_scale, dlse=d_lse)
        except torch.cuda.OutOfMemoryError:
            if not auto:
                raise                      # asked for explicitly: report that its workspace does not fit
            torch.cuda.empty_cache()       # chosen here: the atomic form needs no workspace
    return ops.hash_attn_bwd(q, k, v, lists, off, counts, groups, out.contiguous(),
                             lse.float().contiguous(), d_out.contiguous(), sm_scale, dlse=d_lse)

