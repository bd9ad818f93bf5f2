"""The path as autograd sees it.

* ``torch.ops.notbad.attention_hash_varlen`` with the reference's own operator schema
  (triton_kernel.py:16-22: queries already sorted by bucket, groups given as
  ``q_hashes_z / q_hashes_count / q_hashes_offset``, base-2 LSE out), so the reference's
  host wrapper (triton_kernel.py:51-119) can run on top of it unchanged.  The reference
  registers a backward that returns ``None`` for every input (triton_kernel.py:44-48);
  here ``q``, ``k`` and ``v`` receive gradients from ``fm_hash_attn_bwd*``.
* ``torch.ops.fastmem.attention_hash_varlen``: the same operator on the arguments of the
  Python-level ``attention_hash_varlen`` (queries in their own order, one hash per query,
  natural-log fp32 LSE), differentiable in ``q``, ``k``, ``v`` through ``out`` and ``lse``.
* ``ring_cross_attention_approx``: one ``autograd.Function`` for the whole module forward of
  ``_RingApproxCrossAttentionFunc`` (memory.py:234-418) on one device: centroids, index
  build, query hash, causal local attention, memory attention, LSE merge; the backward
  uses the merged ``out`` / ``lse`` for both parts as the reference does (memory.py:347-418).

The ring send/receive and the collectives of the reference are not part of it.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops
from .hash_attention import _as_i32, attention_hash_varlen_backward

LOG2E = 1.4426950408889634
_NEG = -1e30


# ------------------------------------------------------------------ fastmem::attention_hash_varlen
@torch.library.custom_op("fastmem::attention_hash_varlen", mutates_args=())
def _fm_attention_hash_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_hashes: torch.Tensor,
                              k_hash_counts: torch.Tensor, q_hashes: torch.Tensor,
                              sm_scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    return ops.attention_hash_varlen_i32(q.contiguous(), k.contiguous(), v.contiguous(),
                                         _as_i32(k_hashes).contiguous(), _as_i32(k_hash_counts).contiguous(),
                                         _as_i32(q_hashes).contiguous(), sm_scale)


@_fm_attention_hash_varlen.register_fake
def _(q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale):
    return torch.empty_like(q), q.new_empty(q.shape[:-1], dtype=torch.float32)


def _fm_setup(ctx, inputs, output):
    q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale = inputs
    out, lse = output
    ctx.save_for_backward(q, k, v, k_hashes, k_hash_counts, q_hashes, out, lse)
    ctx.sm_scale = sm_scale


def _fm_backward(ctx, grad_out, grad_lse):
    q, k, v, k_hashes, k_hash_counts, q_hashes, out, lse = ctx.saved_tensors
    if grad_out is None:
        grad_out = torch.zeros_like(out)
    dq, dk, dv = attention_hash_varlen_backward(grad_out.to(q.dtype).contiguous(), q.contiguous(), k.contiguous(),
                                                v.contiguous(), out, lse, k_hashes, k_hash_counts, q_hashes,
                                                ctx.sm_scale, d_lse=grad_lse)
    return dq, dk.to(k.dtype), dv.to(v.dtype), None, None, None, None


_fm_attention_hash_varlen.register_autograd(_fm_backward, setup_context=_fm_setup)


def attention_hash_varlen_op(q, k, v, k_hashes, k_hash_counts, q_hashes, sm_scale):
    """``attention_hash_varlen`` as a registered, differentiable operator: ``(out, lse)`` with the fp32
    natural-log LSE; ``loss.backward()`` reaches ``q``, ``k`` and ``v``."""
    return torch.ops.fastmem.attention_hash_varlen(q, k, v, k_hashes, k_hash_counts, q_hashes, float(sm_scale))


# ------------------------------------------------------------------ notbad::attention_hash_varlen
def _hashes_of_sorted_queries(q_hashes_z, q_hashes_count, batch_size, q_seq_len):
    """The bucket of every query of the sorted layout, from the groups the reference passes
    (triton_kernel.py:81-84: one entry per distinct (row, bucket) pair in (row, bucket) order, ``q_hashes_z``
    its bucket, ``q_hashes_count`` its number of queries; a group never spans two rows)."""
    z = torch.repeat_interleave(q_hashes_z, q_hashes_count, output_size=batch_size * q_seq_len)
    return z.reshape(batch_size, q_seq_len)


@torch.library.custom_op("notbad::attention_hash_varlen", mutates_args=())
def _notbad_attention_hash_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                                  k_hashes: torch.Tensor, k_hash_counts: torch.Tensor, k_hash_offset: torch.Tensor,
                                  q_hashes_z: torch.Tensor, q_hashes_count: torch.Tensor,
                                  q_hashes_offset: torch.Tensor,
                                  sm_scale: float, q_seq_len: int, kv_seq_len: int,
                                  d_head: int, n_buckets: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same schema as the reference's operator (triton_kernel.py:16-22).  ``q`` holds the queries sorted by
    bucket inside every batch row (triton_kernel.py:75-77); the results come back in that order, the LSE in
    base 2 (``lse2 = m + log2(l)``, triton_kernel.py:222), ``-inf`` for a query whose bucket is empty.
    ``k_hash_offset`` and ``q_hashes_offset`` are implied by the counts and not read."""
    batch_size = q.shape[0]
    assert q.shape[1] == q_seq_len and k.shape[1] == kv_seq_len and q.shape[2] == d_head
    qh = _hashes_of_sorted_queries(q_hashes_z, q_hashes_count, batch_size, q_seq_len)
    # grouping a sorted sequence again is the identity permutation (the grouping is stable)
    out, lse = ops.attention_hash_varlen_i32(q.contiguous(), k.contiguous(), v.contiguous(),
                                             _as_i32(k_hashes).contiguous(),
                                             _as_i32(k_hash_counts.reshape(batch_size, n_buckets)).contiguous(),
                                             _as_i32(qh).contiguous(), sm_scale)
    lse2 = torch.where(lse < _NEG, torch.full_like(lse, -float("inf")), lse * LOG2E)
    return out, lse2


@_notbad_attention_hash_varlen.register_fake
def _(q, k, v, k_hashes, k_hash_counts, k_hash_offset, q_hashes_z, q_hashes_count, q_hashes_offset, sm_scale,
      q_seq_len, kv_seq_len, d_head, n_buckets):
    return torch.empty_like(q), q.new_empty(q.shape[:-1], dtype=torch.float32)


def _notbad_setup(ctx, inputs, output):
    (q, k, v, k_hashes, k_hash_counts, _k_off, q_hashes_z, q_hashes_count, _q_off, sm_scale, q_seq_len, _kv,
     _d, n_buckets) = inputs
    out, lse2 = output
    ctx.save_for_backward(q, k, v, k_hashes, k_hash_counts, q_hashes_z, q_hashes_count, out, lse2)
    ctx.sm_scale, ctx.q_seq_len, ctx.n_buckets = sm_scale, q_seq_len, n_buckets


def _notbad_backward(ctx, grad_out, grad_lse2):
    q, k, v, k_hashes, k_hash_counts, q_hashes_z, q_hashes_count, out, lse2 = ctx.saved_tensors
    B = q.shape[0]
    qh = _hashes_of_sorted_queries(q_hashes_z, q_hashes_count, B, ctx.q_seq_len)
    lse = torch.where(torch.isinf(lse2), torch.full_like(lse2, torch.finfo(torch.float32).min), lse2 / LOG2E)
    if grad_out is None:
        grad_out = torch.zeros_like(out)
    d_lse = None if grad_lse2 is None else grad_lse2 * LOG2E          # d loss / d lse = d loss / d lse2 * log2(e)
    dq, dk, dv = attention_hash_varlen_backward(grad_out.to(q.dtype).contiguous(), q.contiguous(), k.contiguous(),
                                                v.contiguous(), out, lse, k_hashes,
                                                k_hash_counts.reshape(B, ctx.n_buckets), qh, ctx.sm_scale,
                                                d_lse=d_lse)
    return (dq, dk.to(k.dtype), dv.to(v.dtype)) + (None,) * 11


_notbad_attention_hash_varlen.register_autograd(_notbad_backward, setup_context=_notbad_setup)


# ------------------------------------------------------------------ local attention backward
_prefix_lists = {}


_PREFIX_CHUNK_ENTRIES = 1 << 24   # list entries per KV head and call of the gathered backward (64 MiB of int32)
_PREFIX_BLOCK = 8                 # tokens that share a bucket: with G query heads a bucket has 8 G queries


def _causal_prefix_lists(H: int, t0: int, t1: int, S: int, L: int, device):
    """Bucket lists that express the causal local attention of tokens t0 .. t1-1 (t0 a multiple of the token
    block) as two gathered ones.  Token t sees keys 0 .. t + (L - S).  *Blocks*: the tokens of a block of
    ``_PREFIX_BLOCK`` share bucket (t - t0) // block, whose list is what the block's first token sees -- keys
    every token of the block sees.  *Diagonal*: token t alone in bucket t - t0, whose list is the rest of its
    keys, the at most block - 1 keys between its block's first token and itself.  The last pair built is kept."""
    key = (H, t0, t1, S, L, str(device))
    if key not in _prefix_lists:
        P = _PREFIX_BLOCK
        off = L - S
        j = torch.arange(L, device=device)
        first = torch.arange(t0, t1, P, device=device)                                       # a block's first token
        lim_b = (first + off + 1).clamp(min=0, max=L)                                        # keys seen by it
        flat_b = j.expand(first.numel(), L)[j[None, :] < lim_b[:, None]].to(torch.int32)     # row-major (block, key)
        cnt_b = lim_b.to(torch.int32).unsqueeze(0).expand(H, first.numel()).contiguous()
        t = torch.arange(t0, t1, device=device)
        lo = ((t - t0) // P * P + t0 + off + 1).clamp(min=0, max=L)                          # first key not in the block's list
        hi = (t + off + 1).clamp(min=0, max=L)
        w = torch.arange(P, device=device)
        keys_d = lo[:, None] + w[None, :]
        flat_d = keys_d[keys_d < hi[:, None]].to(torch.int32)
        cnt_d = (hi - lo).clamp(min=0).to(torch.int32).unsqueeze(0).expand(H, t.numel()).contiguous()
        _prefix_lists.clear()                                                                # one shape at a time
        _prefix_lists[key] = (flat_b.repeat(H), cnt_b, flat_d.repeat(H), cnt_d)
    return _prefix_lists[key]


def local_attention_backward(d_out, q, k, v, out, lse, sm_scale: float, causal: bool = True,
                             staged: Optional[bool] = None):
    """Gradients of the dense local attention (the ``attention_backward(dout, q, k_self, v_self, out, lse,
    sm_scale, True)`` call at memory.py:368, which the reference does not define).  ``q, out, d_out
    [H*G,S,d]``, ``k, v [H,L,d]``, ``lse [H*G,S]``; ``out`` / ``lse`` may be the merged result.  Returns
    ``(dq [H*G,S,d], dk, dv [H,L,d] fp32)``.

    No kernel of its own: given ``out`` and ``lse`` the backward is a sum over keys, so the causal case is two
    backwards of the gathered attention whose key sets partition every token's prefix.  In the first, blocks of
    8 tokens (with all their G query heads: 8 G queries) share a bucket that lists the keys all of them see; in
    the second every token has a bucket of its own with the up to 7 keys left.  The lists of the first hold
    S L / 16 entries per KV head at S = L (one sixteenth of a list per token), taken in token chunks that keep a
    call below 2^24 entries per head; dk and dv add up over the calls, dq is the sum of the two parts (each
    rounded to q's dtype, added in fp32).  Without the causal mask one bucket lists all keys.

    ``staged`` is passed on to :func:`attention_hash_varlen_backward`: ``None`` (the default) takes the form
    without atomics for bf16 with d = 128 where a call has at least as many queries as buckets (results do not
    depend on scheduling) and the atomic adds otherwise or when its workspace does not fit."""
    HG, S, d = q.shape
    H, L, _ = k.shape
    G = HG // H
    dev = q.device
    q4, do4 = q.reshape(H, G, S, d), d_out.reshape(H, G, S, d)
    o4, l4 = out.reshape(H, G, S, d), lse.reshape(H, G, S)
    k, v = k.contiguous(), v.contiguous()
    if not causal:
        flat = torch.arange(L, device=dev, dtype=torch.int32).repeat(H)
        cnt = torch.full((H, 1), L, dtype=torch.int32, device=dev)
        qh = torch.zeros(H, G * S, dtype=torch.int32, device=dev)
        flat3 = lambda x: x.reshape(H, G * S, *x.shape[3:]).contiguous()
        dq, dk, dv = attention_hash_varlen_backward(flat3(do4), flat3(q4), k, v, flat3(o4).to(q.dtype), flat3(l4).float(),
                                                    flat, cnt, qh, sm_scale, staged=staged)
        return dq.reshape(HG, S, d), dk, dv
    P = _PREFIX_BLOCK
    T = max(64, min(S, _PREFIX_CHUNK_ENTRIES * P // max(L, 1))) // P * P        # tokens per chunk, whole blocks
    dq = torch.empty((H, G, S, d), dtype=q.dtype, device=dev)
    dk = dv = None
    for t0 in range(0, S, T):
        t1 = min(S, t0 + T)
        n = t1 - t0
        flat_b, cnt_b, flat_d, cnt_d = _causal_prefix_lists(H, t0, t1, S, L, dev)
        t = torch.arange(n, device=dev, dtype=torch.int32)
        sl = lambda x: x[:, :, t0:t1].reshape(H, G * n, *x.shape[3:]).contiguous()
        args = (sl(do4), sl(q4), k, v, sl(o4).to(q.dtype), sl(l4).float())
        dq_c = None
        for flat, cnt, bucket_of in ((flat_b, cnt_b, t // P), (flat_d, cnt_d, t)):
            if flat.numel() == 0:                                                   # a single token has no diagonal
                continue
            qh = bucket_of.repeat(H * G).reshape(H, G * n)                         # query g*n + t -> its bucket
            dq_p, dk_p, dv_p = attention_hash_varlen_backward(*args, flat, cnt, qh, sm_scale, staged=staged)
            dq_c = dq_p.float() if dq_c is None else dq_c + dq_p.float()
            dk, dv = (dk_p, dv_p) if dk is None else (dk + dk_p, dv + dv_p)
        dq[:, :, t0:t1] = 0 if dq_c is None else dq_c.to(q.dtype).reshape(H, G, n, d)
    if dk is None:                                                                  # no token sees a key
        dk, dv = (torch.zeros((H, L, d), dtype=torch.float32, device=dev) for _ in range(2))
    return dq.reshape(HG, S, d), dk, dv


# ------------------------------------------------------------------ the module forward as one Function
class _ApproxCrossAttentionFunc(torch.autograd.Function):
    """``_RingApproxCrossAttentionFunc`` (memory.py:234-418) with a world of one: no all-reduce, all-to-all,
    all-gather or ring steps; the key window is all of ``k``."""

    @staticmethod
    def forward(ctx, q, kq, k_self, v_self, k, v, rnd_centroids, sm_scale, n_hashes, n_results, centroid_topk):
        from .memory import Memory, compute_centroids, update_out_and_lse
        batch_size, n_heads, seq_len, d_qkv = q.shape
        assert batch_size == 1
        _, k_heads, context_len, _ = k.shape
        n_groups = n_heads // k_heads
        assert n_heads % k_heads == 0, f'{q.shape} == {k.shape}'
        assert kq.shape[0] == k_self.shape[0] == k.shape[0] == batch_size
        assert rnd_centroids.shape[0] == n_hashes
        # memory.py:252-258: top-k-mean centroids, (all-reduce over one rank,) L2-normalised; [C,H,d] -> [H,C,d]
        centroids = compute_centroids(kq[0], rnd_centroids, n_hashes, n_groups, centroid_topk, normalize=True)
        A = centroids.permute(1, 0, 2).contiguous()
        mem = Memory.build(k[0], v[0], A, min(int(n_results), context_len))                 # memory.py:260-278
        q3 = q[0].reshape(k_heads, n_groups * seq_len, d_qkv).contiguous()
        q_hashes = mem.hash(q3)                                                             # memory.py:280-283
        block_out, block_lse = ops.local_attn_fwd(q[0].contiguous(), k_self[0].contiguous(), v_self[0].contiguous(),
                                                  sm_scale, True)                           # memory.py:302-304
        out, lse = update_out_and_lse(None, None, block_out.reshape(q3.shape), block_lse.reshape(k_heads, -1))
        mo, ml = mem.attend(q3, sm_scale, q_hash=q_hashes)                                  # memory.py:319-321
        out, lse = update_out_and_lse(out.contiguous(), lse.contiguous(), mo, ml)           # memory.py:332
        out = out.to(q.dtype)
        ctx.sm_scale = sm_scale
        # Everything the backward reads goes through save_for_backward (the reference keeps clones, k_og / v_og,
        # memory.py:243-244): k and v themselves, so that an in-place update of the memory between forward and
        # backward (a KV cache that is appended to or overwritten) is caught by autograd's version counter
        # instead of silently giving gradients against the new contents, and the bucket lists with their
        # key-ordered copy, from which the backward rebuilds a Memory view without building an index again.
        attn_idx = mem._attn_idx if mem._attn_idx is not None else mem.bucket_idx.new_empty(0)
        ctx.save_for_backward(q, k_self, v_self, q_hashes, out, lse.squeeze(-1), k, v, A, mem.bucket_idx, attn_idx)
        ctx.mark_non_differentiable(q_hashes)
        return out.reshape(q.shape), q_hashes

    @staticmethod
    def backward(ctx, dout, _d_hashes):
        from .memory import Memory
        q, k_self, v_self, q_hashes, out, lse, k, v, A, bucket_idx, attn_idx = ctx.saved_tensors
        sm_scale = ctx.sm_scale
        mem = Memory(k[0], v[0], A, bucket_idx)
        if attn_idx.numel():
            mem._attn_idx = attn_idx
        _, n_heads, seq_len, d_qkv = q.shape
        k_heads = k_self.shape[1]
        dout3 = dout[0].to(q.dtype).reshape(out.shape).contiguous()
        q3 = q[0].reshape(out.shape).contiguous()
        # memory.py:367-369: the local part, with the merged out / lse
        dq, dk_self, dv_self = local_attention_backward(dout[0].to(q.dtype).contiguous(), q[0].contiguous(),
                                                        k_self[0], v_self[0], out.reshape(n_heads, seq_len, d_qkv),
                                                        lse.reshape(n_heads, seq_len), sm_scale, True)
        # memory.py:386-393: the memory part
        mq, dk, dv = mem.attend_backward(dout3, q3, out, lse, sm_scale, q_hash=q_hashes)
        dq = dq.float() + mq.reshape(n_heads, seq_len, d_qkv).float()
        cast = lambda t, like: t.to(like.dtype).reshape(like.shape)
        return (cast(dq, q), None, cast(dk_self, k_self), cast(dv_self, v_self), cast(dk, mem.keys.unsqueeze(0)),
                cast(dv, mem.values.unsqueeze(0)), None, None, None, None, None)


def ring_cross_attention_approx(q, kq, k_self, v_self, k, v, rnd_centroids, sm_scale, n_hashes, n_results, *,
                                centroid_topk: int, sampling_method: Optional[str] = None,
                                return_hashes: bool = False):
    """Drop-in for ``ring_cross_attention_approx`` (memory.py:421-425) on one device.

    :param q: ``[1, n_heads, seq_len, d]``
    :param kq: ``[1, n_heads, context_len, d]`` key queries the centroids are built from (memory.py:252)
    :param k_self, v_self: ``[1, k_heads, seq_len, d]`` local keys / values (causal)
    :param k, v: ``[1, k_heads, context_len, d]`` the memory
    :param rnd_centroids: ``[n_hashes, d]`` initial centroids (memory.py:489-493)
    :param centroid_topk: the reference's ``consts.centroid_topk`` (memory.py:220)
    :return: ``out [1, n_heads, seq_len, d]`` in q's dtype; differentiable in ``q``, ``k_self``, ``v_self``,
        ``k`` and ``v`` (``kq`` and the centroids receive no gradient, memory.py:418).
    """
    out, hashes = _ApproxCrossAttentionFunc.apply(q, kq, k_self, v_self, k, v, rnd_centroids, float(sm_scale),
                                                  int(n_hashes), int(n_results), int(centroid_topk))
    return (out, hashes) if return_hashes else out
