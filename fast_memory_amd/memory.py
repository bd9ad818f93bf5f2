"""Module-level API of the indexed memory (the reference's memory.py), on one
MI355X: LSE merge, construction of the projection matrix, the per-window
attention step, and the ``Memory`` object the README describes (build a memory
from past keys, query it, get attention output plus log-sum-exp).

Ring send/receive, collectives, the autograd wrapper and the model hook of the
reference are not part of this package.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from . import ops
from .hash_attention import attention_hash_varlen


# --------------------------------------------------------------------------
def update_out_and_lse(out: Optional[torch.Tensor], lse: Optional[torch.Tensor],
                       block_out: torch.Tensor, block_lse: torch.Tensor
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for ``update_out_and_lse`` (memory.py:54-71): merges a partial
    attention into the running fp32 ``(out, lse[..., None])`` pair, in place."""
    if out is None:
        return block_out.to(torch.float32), block_lse.to(torch.float32).unsqueeze(dim=-1)
    assert out.dtype == torch.float32 and lse.dtype == torch.float32
    assert out.is_contiguous() and lse.is_contiguous()
    ops.lse_merge_(out, lse, block_out.contiguous(), block_lse.to(torch.float32).contiguous())
    return out, lse


# --------------------------------------------------------------------------
_init_cache = {}


def init_centroids(n_buckets: int, d: int, device, dtype) -> torch.Tensor:
    """The reference's initial centroids (memory.py:489-493).  The seeded host draw and its upload cost a few
    milliseconds, more than a K-means fit of 2 M keys: the tensor is kept per (shape, device, dtype) and a
    copy is handed out."""
    key = (int(n_buckets), int(d), str(torch.device(device)), dtype)
    if key not in _init_cache:
        rng = np.random.RandomState(42)
        _init_cache[key] = torch.tensor(rng.randn(n_buckets, d), device=device, dtype=dtype, requires_grad=False)
    return _init_cache[key].clone()


@torch.no_grad()
def compute_centroids(kq: torch.Tensor, centroids: torch.Tensor, n_hashes: int, n_groups: int,
                      centroid_topk: int, normalize: bool = False) -> torch.Tensor:
    """Drop-in for ``compute_centroids`` (memory.py:209-231); ``centroid_topk``
    replaces the reference's module-global ``consts.centroid_topk``.

    ``kq [H*G, N, d]``, ``centroids [C, d]`` -> ``[C, H, d]``.  With
    ``normalize`` the rows are L2-normalised as the caller does at
    memory.py:258 (the all-reduce before it is the identity on one device)."""
    n_heads, context_len, d_qkv = kq.shape
    k_heads = n_heads // n_groups
    assert centroids.shape == (n_hashes, d_qkv)
    kq_hash = ops.l2_normalize(kq.contiguous(), 1e-6)
    # scores[hg, c, i] = centroids[c] . kq_hash[hg, i]; rows ordered (hg, c)
    A = centroids.to(kq.dtype).unsqueeze(0).expand(n_heads, -1, -1).contiguous()
    top = ops.build_index(A, kq_hash, centroid_topk)                 # [HG, C, k]
    top = top.permute(1, 0, 2).contiguous()                          # [C, HG, k]
    return ops.topk_mean(kq_hash, top, k_heads, n_groups, normalize=normalize)


@torch.no_grad()
def kmeans_spherical(X: torch.Tensor, init: torch.Tensor, iters: int, normalize_rows: Optional[float] = None):
    """Spherical K-means (README.md:37-45): ``X [H,N,d]`` unit rows, ``init
    [H,C,d]`` -> centroids ``[H,C,d]`` (unit rows) and the labels of the last
    assignment ``[H,N]`` int32.  With ``normalize_rows=eps`` X holds rows of any length and the
    result is that of K-means on ``x / max(|x|, eps)``: the assignment ``argmax_c c.x`` does not depend
    on ``|x|``, and the update divides every member by its norm as it adds it."""
    cent = init.contiguous()
    C = cent.shape[1]
    labels = None
    for _ in range(iters):
        labels = ops.qhash(cent, X)
        groups = ops.group_queries(labels, C)
        cent = ops.segment_mean(X, groups, cent, normalize_rows)
    return cent, labels


def fit_projection(keys: torch.Tensor, n_buckets: int, iters: int = 2,
                   init: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A ``[H,C,d]`` from ``iters`` spherical K-means iterations on the
    L2-normalised keys ``[H,N,d]`` (README.md:33-45), starting from the
    reference's seeded random centroids, normalised."""
    H, N, d = keys.shape
    if init is None:
        c0 = init_centroids(n_buckets, d, keys.device, torch.float32)
        c0 = (c0 / c0.norm(dim=-1, keepdim=True)).to(keys.dtype)
        init = c0.unsqueeze(0).expand(H, -1, -1).contiguous()
    # no normalised copy of the keys is made: see kmeans_spherical
    cent, _ = kmeans_spherical(keys.contiguous(), init, iters, normalize_rows=1e-6)
    return cent


# --------------------------------------------------------------------------
def ring_attention_masked_forward(k_hashes, q_hashes, q, k, v, sm_scale, rank,
                                  lse_dtype: Optional[torch.dtype] = torch.float32):
    """Drop-in for ``ring_attention_masked_forward`` (memory.py:106-163).

    :param k_hashes: ``[n_buckets, k_heads, bucket_size]`` global key indices
    :param q_hashes: ``[k_heads, n_groups, seq_len]``
    :param q: ``[1, n_heads, seq_len, d]``
    :param k, v: ``[1, k_heads, context_len, d]`` -- the window of keys with
        global indices ``[rank*context_len, (rank+1)*context_len)``
    :return: ``(out [1,n_heads,seq_len,d], lse [1,n_heads,seq_len])``; the
        LSE is fp32 unless ``lse_dtype=None`` asks for the reference's rounding
        to q's dtype.
    """
    batch_size, n_heads, seq_len, d_head = q.shape
    _, k_heads, context_len, _ = k.shape
    n_groups = n_heads // k_heads
    assert batch_size == 1
    assert k_hashes.shape[1] == k_heads
    assert q_hashes.shape[0] == k_heads
    assert q_hashes.shape[1] == n_groups
    assert q_hashes.shape[2] == seq_len
    assert k_hashes.numel() > 0, k_hashes.shape

    kh = k_hashes.permute(1, 0, 2).to(torch.int32).contiguous()     # H C Z
    flat, counts, _ = ops.window_filter(kh, rank * context_len, (rank + 1) * context_len)
    out, lse = attention_hash_varlen(q.reshape(k_heads, -1, d_head), k.reshape(k_heads, -1, d_head),
                                     v.reshape(k_heads, -1, d_head), flat, counts,
                                     q_hashes.reshape(k_heads, -1), sm_scale, lse_dtype=lse_dtype)
    return out.reshape(batch_size, n_heads, seq_len, d_head), lse.reshape(batch_size, n_heads, seq_len)


# --------------------------------------------------------------------------
@torch.no_grad()
def calc_ref_centroids(q_self: torch.Tensor, k: torch.Tensor, topk: int = 128,
                       workspace_bytes: int = 2 << 30) -> torch.Tensor:
    """Drop-in for ``calc_ref_centroids`` (memory.py:428-456): the target of the learned projection.

    For every query the ``topk`` keys with the largest scores ``q.k`` are found (value descending, key
    index ascending; the reference's ``torch.topk`` leaves ties unspecified and ranks scores rounded to
    q's dtype, here the fp32 scores are ranked); every key's centroid is the sum of the queries that
    selected it, divided by ``topk`` and by its norm clamped at 1e-6.

    :param q_self: ``[batch, n_heads, seq_len, d]``
    :param k: ``[batch, k_heads, context_len, d]``
    :return: ``[batch, k_heads, n_groups, context_len, d]`` in q's dtype
    """
    batch_size, n_heads, seq_len, d_qkv = q_self.shape
    _, k_heads, context_len, _ = k.shape
    n_groups = n_heads // k_heads
    _topk = min(topk, context_len)
    rows = batch_size * k_heads
    qa = q_self.reshape(rows, n_groups * seq_len, d_qkv).contiguous()
    top = ops.build_index(qa, k.reshape(rows, context_len, d_qkv).contiguous(), _topk)   # [rows, G*S, topk]
    labels = top.reshape(rows * n_groups, seq_len * _topk)
    X = q_self.reshape(rows * n_groups, seq_len, d_qkv).contiguous()
    sums = torch.empty((rows * n_groups, context_len, d_qkv), dtype=torch.float32, device=q_self.device)
    # the grouping's table is (blocks of 256 entries) x context_len ints per row: bound it
    per_row = ((seq_len * _topk + 255) // 256) * context_len * 4
    step = max(1, workspace_bytes // max(per_row, 1))
    for r0 in range(0, rows * n_groups, step):
        r1 = min(rows * n_groups, r0 + step)
        g = ops.group_queries(labels[r0:r1].contiguous(), context_len)
        members = torch.div(g.q_perm, _topk, rounding_mode="floor").to(torch.int32)   # entry -> its query
        sums[r0:r1] = ops.segment_sum(X[r0:r1].contiguous(), members, g.bin_off, g.bin_count)
    cent = sums / _topk
    cent = cent / cent.norm(p=2, dim=-1, keepdim=True).clamp(min=1e-6)
    return cent.to(q_self.dtype).reshape(batch_size, k_heads, n_groups, context_len, d_qkv)


def learn_emb_proj(kq: torch.Tensor, q_self: torch.Tensor, k: torch.Tensor):
    """Drop-in for ``learn_emb_proj`` (memory.py:459-484) without its logging: normalised ``kq`` and the
    MSE between it and :func:`calc_ref_centroids`.

    :param kq: ``[batch, context_len, n_heads * d]``
    :return: ``(kq [batch, n_heads, context_len, d] normalised, loss)``"""
    batch_size, n_heads, seq_len, d_qkv = q_self.shape
    _, k_heads, context_len, _ = k.shape
    n_groups = n_heads // k_heads
    kq = kq.view(*kq.shape[:2], n_heads, d_qkv).permute(0, 2, 1, 3).contiguous()
    kq = kq.reshape(batch_size, k_heads, n_groups, -1, d_qkv)
    kq = kq / torch.norm(kq, p=2, dim=-1, keepdim=True).clamp(min=1e-6)
    with torch.no_grad():
        centroids = calc_ref_centroids(q_self, k)
    assert list(kq.shape) == list(centroids.shape), f'{kq.shape} != {centroids.shape}'
    return kq.reshape(batch_size, n_heads, -1, d_qkv), torch.nn.functional.mse_loss(kq, centroids)


# --------------------------------------------------------------------------
def ring_attention_masked_backward(k_hashes, q_hashes, h_idx, d_out, q, k, v, out, softmax_lse, sm_scale, rank):
    """Drop-in for ``ring_attention_masked_backward`` (memory.py:166-206) on one window of keys.

    Same arguments and layouts as the reference (``h_idx`` is accepted and unused: the head index is
    implied by the layout); ``out`` / ``softmax_lse`` are the final (merged) results.  The reference
    materialises the dense ``[S, N]`` probabilities; here every query only visits its bucket's keys.

    :return: ``(dQ [1,n_heads,seq_len,d], dK, dV [1,k_heads,context_len,d])`` in q's dtype.
    """
    from .hash_attention import attention_hash_varlen_backward
    batch_size, n_heads, seq_len, d_head = q.shape
    _, k_heads, context_len, _ = k.shape
    assert batch_size == 1 and n_heads % k_heads == 0
    kh = k_hashes.permute(1, 0, 2).to(torch.int32).contiguous()     # H C Z
    flat, counts, _ = ops.window_filter(kh, rank * context_len, (rank + 1) * context_len)
    dq, dk, dv = attention_hash_varlen_backward(
        d_out.reshape(k_heads, -1, d_head).contiguous(), q.reshape(k_heads, -1, d_head).contiguous(),
        k.reshape(k_heads, -1, d_head), v.reshape(k_heads, -1, d_head), out.reshape(k_heads, -1, d_head),
        softmax_lse.reshape(k_heads, -1).float(), flat, counts, q_hashes.reshape(k_heads, -1), sm_scale)
    return (dq.reshape(q.shape), dk.to(k.dtype).reshape(k.shape), dv.to(v.dtype).reshape(v.shape))


# --------------------------------------------------------------------------
class Memory:
    """Indexed memory over one sequence's past keys (README.md:5-7).

    ``keys, values [H,N,d]``; ``A [H,C,d]`` projection rows; ``Z`` bucket
    capacity.  ``attend`` returns the attention over the hashed bucket and its
    log-sum-exp so the caller can merge it with attention over other keys
    (``merge`` / ``update_out_and_lse``).

    ``bucket_idx [H,C,L]`` are the lists as ``torch.topk`` orders them (memory.py:273, descending score).
    With ``key_order`` (the default) the attention and its backward read a copy in ascending key order,
    made the first time a call brings at least one query per bucket and kept until the lists change: the
    result of the gathered softmax does not depend on the order of a list, the speed of the row gathers
    does (:func:`ops.lists_key_order`).
    """

    def __init__(self, keys: torch.Tensor, values: torch.Tensor, A: torch.Tensor, bucket_idx: torch.Tensor,
                 bucket_val: Optional[torch.Tensor] = None, Z: Optional[int] = None, key_order: bool = True):
        self.keys, self.values, self.A = keys, values, A
        self.Z = int(Z) if Z is not None else bucket_idx.shape[2]       # capacity; lists are shorter while N < Z
        self.key_order = bool(key_order)
        self._build_status = None      # the status word of a build whose check was deferred (check_build)
        self._set_lists(bucket_idx, bucket_val)

    def _set_lists(self, bucket_idx: torch.Tensor, bucket_val: Optional[torch.Tensor]):
        self.bucket_idx, self.bucket_val = bucket_idx.contiguous(), bucket_val
        self._inverse = None
        self._attn_idx = None
        H, C, L = bucket_idx.shape
        dev = bucket_idx.device
        self.bucket_cnt = torch.full((H, C), L, dtype=torch.int32, device=dev)
        self.bucket_off = (torch.arange(H * C, dtype=torch.int64, device=dev) * L).reshape(H, C)

    @classmethod
    def build(cls, keys: torch.Tensor, values: torch.Tensor, A: torch.Tensor, Z: int,
              workspace_bytes: int = 8 << 30, keep_values: bool = False, key_order: bool = True,
              defer_check: bool = False) -> "Memory":
        """``keep_values`` also stores the projections of the listed keys (4 bytes per list entry), which
        :meth:`append` needs; ``key_order`` as in the class description.  The fused build's only host
        synchronisation is the read-back of its status word; with ``defer_check`` the build returns without
        it (build and attention can then be queued back to back, or recorded into one graph) and
        :meth:`check_build` -- called by :meth:`append` and :meth:`save`, or by the caller at a point where
        waiting costs nothing -- looks at the word and rebuilds the lists if rows were left unresolved."""
        keys, values, A = keys.contiguous(), values.contiguous(), A.contiguous()
        assert keys.shape == values.shape and A.shape[0] == keys.shape[0] and A.shape[2] == keys.shape[2]
        res = ops.build_index(A, keys, Z, workspace_bytes, return_values=keep_values, defer_check=defer_check)
        res = res if isinstance(res, tuple) else (res,)
        status = res[-1] if defer_check else None
        idx = res[0]
        val = res[1] if keep_values else None
        mem = cls(keys, values, A, idx, val, Z, key_order)
        mem._build_status = status
        mem._workspace_bytes = workspace_bytes
        return mem

    def check_build(self) -> bool:
        """Reads the status word a deferred build left (synchronises with its stream).  ``True``: the lists
        are final.  ``False``: rows had been left unresolved; the lists have now been rebuilt by the unfused
        build, and results computed from them before this call are to be discarded."""
        status, self._build_status = self._build_status, None
        if status is None or status.unresolved() == 0:
            return True
        ops.build_index_unfused_(self.A, self.keys, self.Z, self.bucket_idx, self.bucket_val,
                                 getattr(self, "_workspace_bytes", 8 << 30))
        self._inverse = None
        self._attn_idx = None
        return False

    def append(self, new_keys: torch.Tensor, new_values: torch.Tensor, workspace_bytes: int = 8 << 30) -> "Memory":
        """Add keys/values ``[H,M,d]`` at the end of the memory and bring the bucket lists to what a rebuild
        over all keys would give, without projecting the old keys again (the reference rebuilds on every
        forward, memory.py:252-278).  Needs ``build(..., keep_values=True)``.  Returns ``self``."""
        assert self.bucket_val is not None, "Memory.build(..., keep_values=True) is needed to append"
        self.check_build()
        new_keys, new_values = new_keys.contiguous(), new_values.contiguous()
        H, M, d = new_keys.shape
        assert new_values.shape == new_keys.shape and H == self.keys.shape[0] and d == self.keys.shape[2]
        n_old = self.keys.shape[1]
        full = n_old >= self.Z        # full lists are updated in place: buckets that take no new key stay untouched
        res = ops.index_append(self.A, new_keys, n_old, self.bucket_idx, self.bucket_val, self.Z, inplace=full)
        self.keys = torch.cat([self.keys, new_keys], dim=1)
        self.values = torch.cat([self.values, new_values], dim=1)
        if res is None:       # a bucket took more new keys than the merge holds: rebuild
            res = ops.build_index(self.A, self.keys, self.Z, workspace_bytes, return_values=True)
        if res[0] is not self.bucket_idx:
            self._set_lists(*res)
        self._inverse = None          # the lists changed (possibly in place)
        self._attn_idx = None
        return self

    def save(self, path: str) -> None:
        """Write the memory (keys, values, A, lists and, if kept, their values) as a safetensors file."""
        from safetensors.torch import save_file
        self.check_build()
        t = {"keys": self.keys, "values": self.values, "A": self.A, "bucket_idx": self.bucket_idx}
        if self.bucket_val is not None:
            t["bucket_val"] = self.bucket_val
        save_file({k: v.contiguous().cpu() for k, v in t.items()}, path, metadata={"Z": str(self.Z), "format": "1"})

    @classmethod
    def load(cls, path: str, device="cuda") -> "Memory":
        """Read a memory written by :meth:`save`; no index is rebuilt."""
        from safetensors import safe_open
        with safe_open(path, framework="pt", device="cpu") as f:
            meta = f.metadata() or {}
            t = {k: f.get_tensor(k).to(device) for k in f.keys()}
        return cls(t["keys"], t["values"], t["A"], t["bucket_idx"], t.get("bucket_val"), int(meta.get("Z", 0)) or None)

    @property
    def n_buckets(self) -> int:
        return self.A.shape[1]

    def hash(self, q: torch.Tensor) -> torch.Tensor:
        """q ``[H,Sq,d]`` -> bucket ids ``[H,Sq]`` int32."""
        return ops.qhash(self.A, q.contiguous())

    def attention_lists(self, n_queries: int = 0) -> torch.Tensor:
        """The flat lists the attention reads: the copy in ascending key order once it exists; a call with at
        least one query per bucket (``n_queries >= C``) makes it, fewer queries do not repay the reordering
        and read ``bucket_idx`` as it is."""
        if self._attn_idx is None and self.key_order and n_queries >= self.n_buckets:
            self._attn_idx = ops.lists_key_order(self.bucket_idx.reshape(-1), self.bucket_off.reshape(-1),
                                                 self.bucket_cnt.reshape(-1), self.keys.shape[1])
            self._inverse = None      # positions in the lists changed
        return self._attn_idx if self._attn_idx is not None else self.bucket_idx.reshape(-1)

    def attend(self, q: torch.Tensor, sm_scale: float, q_hash: Optional[torch.Tensor] = None):
        """q ``[H,Sq,d]`` (Sq = G*S, query head h*G+g) -> ``(out [H,Sq,d], lse [H,Sq] fp32)``."""
        q = q.contiguous()
        if q_hash is None:
            q_hash = self.hash(q)
        groups = ops.group_queries(q_hash, self.n_buckets)
        return ops.hash_attn_fwd(q, self.keys, self.values, self.attention_lists(q.shape[1]), self.bucket_off,
                                 self.bucket_cnt, groups, sm_scale)

    def inverse_index(self) -> "ops.InverseIndex":
        """For every key the positions of :meth:`attention_lists` that name it (kept until those change); the
        backward without atomics sums a key's gradient contributions over them."""
        if getattr(self, "_inverse", None) is None:
            self._inverse = ops.inverse_index(self.attention_lists(), self.bucket_off, self.bucket_cnt,
                                              self.keys.shape[1])
        return self._inverse

    def attend_backward(self, d_out: torch.Tensor, q: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
                        sm_scale: float, q_hash: Optional[torch.Tensor] = None, staged: Optional[bool] = None):
        """Gradients of :meth:`attend` (memory.py:166-206 on the gathered pairs): ``(dq [H,Sq,d], dk, dv
        [H,N,d] fp32)`` for ``d_out [H,Sq,d]``; ``out`` / ``lse`` are the forward's results or the ones merged
        with the local attention (the gradients are then the memory's share).  ``staged`` as in
        ``attention_hash_varlen_backward``; the staged form reuses :meth:`inverse_index`."""
        q = q.contiguous()
        if q_hash is None:
            q_hash = self.hash(q)
        groups = ops.group_queries(q_hash, self.n_buckets)
        lists = self.attention_lists(q.shape[1])
        can_stage = q.dtype in (torch.bfloat16, torch.float16) and q.shape[2] in (64, 128)
        auto = staged is None
        if auto:
            staged = can_stage and q.shape[1] >= self.n_buckets and not ops.generic_kernels_forced()
        args = (out.to(q.dtype).contiguous(), lse.float().contiguous(), d_out.to(q.dtype).contiguous(), sm_scale)
        if staged:
            try:
                return ops.hash_attn_bwd_staged(q, self.keys, self.values, lists, self.bucket_off, self.bucket_cnt,
                                                groups, self.inverse_index(), *args)
            except torch.cuda.OutOfMemoryError:
                if not auto:
                    raise                  # asked for explicitly: report that its workspace does not fit
                torch.cuda.empty_cache()   # chosen here: the atomic form needs no workspace
        return ops.hash_attn_bwd(q, self.keys, self.values, lists, self.bucket_off, self.bucket_cnt, groups, *args)

    def attend_with_local(self, q: torch.Tensor, k_local: torch.Tensor, v_local: torch.Tensor,
                          sm_scale: float, n_groups: int, causal: bool = True):
        """Memory attention LSE-merged with dense attention over local keys
        (memory.py:302-305, 319-332).  q ``[H,G*S,d]`` with ``G = n_groups``;
        k_local, v_local ``[H,L,d]``.  Returns fp32 ``(out [H,G*S,d], lse
        [H,G*S])``."""
        H, Sq, d = q.shape
        S = Sq // n_groups
        q = q.contiguous()
        lo, ll = ops.local_attn_fwd(q.reshape(H * n_groups, S, d), k_local.contiguous(),
                                    v_local.contiguous(), sm_scale, causal)
        out, lse = update_out_and_lse(None, None, lo.reshape(H, Sq, d), ll.reshape(H, Sq))
        mo, ml = self.attend(q, sm_scale)
        out, lse = update_out_and_lse(out.contiguous(), lse.contiguous(), mo, ml)
        return out, lse.squeeze(-1)


class MemoryBatch:
    """A decode batch of memories with different N, C and Z (one per sequence).

    All rows (sequence, KV head) are packed back to back so that one launch
    hashes every query and attends its bucket: ``attend(q)`` with
    ``q [n_seq, H, G, d]`` (one token per query head) returns ``(out
    [n_seq,H,G,d], lse [n_seq,H,G] fp32, hashes [n_seq,H,G])``.  bf16, d=128.
    """

    def __init__(self, memories):
        mems = list(memories)
        assert mems and all(m.keys.dtype == torch.bfloat16 and m.keys.shape[2] == 128 for m in mems)
        self.n_seq, self.H = len(mems), mems[0].keys.shape[0]
        dev = mems[0].keys.device
        # row order (sequence, head)
        self.A_all = torch.cat([m.A.reshape(-1, 128) for m in mems])
        self.K_all = torch.cat([m.keys.reshape(-1, 128) for m in mems])
        self.V_all = torch.cat([m.values.reshape(-1, 128) for m in mems])
        self.idx_all = torch.cat([m.bucket_idx.reshape(-1) for m in mems])
        rows = []
        a = k = i = 0
        for m in mems:
            H, C, Z = m.bucket_idx.shape
            N = m.keys.shape[1]
            for _ in range(H):
                rows.append([a, k, i, N | (C << 32), Z])
                a, k, i = a + C, k + N, i + C * Z
        # descriptors go longest lists first (a workgroup's time grows with Z, and the launch then ends
        # evenly); each names the row of q / out it belongs to (fm_rowdesc.q_row1 = row + 1)
        order = sorted(range(len(rows)), key=lambda r: -rows[r][4])
        rows = [rows[r][:4] + [rows[r][4] | ((r + 1) << 32)] for r in order]
        self.desc = torch.tensor(rows, dtype=torch.int64, device=dev)
        self.shapes = [(m.keys.shape[1], m.bucket_idx.shape[1], m.bucket_idx.shape[2]) for m in mems]

    def attend(self, q: torch.Tensor, sm_scale: float, return_scores: bool = False):
        n_seq, H, G, d = q.shape
        assert n_seq == self.n_seq and H == self.H
        res = ops.decode_hash_attn(q.reshape(n_seq * H, G, d).contiguous(), self.A_all, self.K_all, self.V_all,
                                   self.idx_all, self.desc, sm_scale, return_scores)
        out, lse, h = res[0].reshape(n_seq, H, G, d), res[1].reshape(n_seq, H, G), res[2].reshape(n_seq, H, G)
        return (out, lse, h, res[3]) if return_scores else (out, lse, h)

    def attend_with_local(self, q, k_local, v_local, sm_scale: float):
        """Merged with dense attention over each sequence's local keys ``[n_seq,H,L,d]`` (the single
        query token sees all of them).  Returns fp32 ``(out [n_seq,H,G,d], lse [n_seq,H,G])``."""
        n_seq, H, G, d = q.shape
        L = k_local.shape[2]
        mo, ml, _ = self.attend(q, sm_scale)
        lo, ll = ops.local_attn_fwd(q.reshape(n_seq * H * G, 1, d).contiguous(),
                                    k_local.reshape(n_seq * H, L, d).contiguous(),
                                    v_local.reshape(n_seq * H, L, d).contiguous(), sm_scale, True)
        out, lse = update_out_and_lse(None, None, lo.reshape(n_seq, H, G, d), ll.reshape(n_seq, H, G))
        out, lse = update_out_and_lse(out.contiguous(), lse.contiguous(), mo, ml)
        return out, lse.squeeze(-1)


def merge(out_a, lse_a, out_b, lse_b):
    """Functional LSE merge of two partial attentions (memory.py:54-71)."""
    out, lse = update_out_and_lse(None, None, out_a, lse_a)
    out, lse = update_out_and_lse(out.clone().contiguous(), lse.clone().contiguous(), out_b, lse_b)
    return out, lse.squeeze(-1)
