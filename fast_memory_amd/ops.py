"""Tensor-level wrappers over the C ABI: shape/dtype checks, output and
workspace allocation (torch owns device memory and streams), one C call each."""
from __future__ import annotations

from typing import NamedTuple, Optional, Tuple

import ctypes

import torch

from . import _lib
from ._lib import check

_DT = {torch.float32: _lib.FM_F32, torch.bfloat16: _lib.FM_BF16, torch.float16: _lib.FM_F16}


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise TypeError(f"unsupported dtype {t.dtype}; libfastmem takes float32, bfloat16 and float16")
    return _DT[t.dtype]


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


_no_entries = {}


def _pl(k_idx: torch.Tensor):
    """Pointer to flat bucket lists.  Lists without a single entry (every count zero: all buckets empty, e.g.
    behind a window that no key passes) are an empty tensor, whose data pointer is null, which the library
    refuses; it reads no entry of such lists, so any valid address serves."""
    if k_idx.numel() > 0:
        return k_idx.data_ptr()
    dev_key = (k_idx.device.type, k_idx.device.index)
    if dev_key not in _no_entries:
        _no_entries[dev_key] = torch.zeros(4, dtype=torch.int32, device=k_idx.device)
    return _no_entries[dev_key].data_ptr()


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def _dev(*ts: torch.Tensor) -> None:
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("libfastmem operators take GPU tensors only (there is no CPU path)")
        if not t.is_contiguous():
            raise AssertionError("tensor must be contiguous")


def _ws(nbytes: int, like: torch.Tensor) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=like.device)


# --------------------------------------------------------------------- a1
def project(A: torch.Tensor, K: torch.Tensor) -> torch.Tensor:
    """Y[h,c,n] = sum_d A[h,c,d] K[h,n,d], fp32 (memory.py:261)."""
    _dev(A, K)
    H, C, d = A.shape
    H2, N, d2 = K.shape
    assert H == H2 and d == d2 and A.dtype == K.dtype
    Y = torch.empty((H, C, N), dtype=torch.float32, device=A.device)
    check(_lib.load().fm_project(_p(A), _p(K), _p(Y), H, C, N, d, N, _dt(A), _stream(A)))
    return Y


# --------------------------------------------------------------------- a2
def argtopz(Y: torch.Tensor, Z: int, return_values: bool = False):
    """Indices of the min(Z,N) largest entries per row: value desc, index asc (memory.py:273);
    with ``return_values`` also the values in that order."""
    _dev(Y)
    assert Y.dtype == torch.float32
    N = Y.shape[-1]
    rows = Y.numel() // N if N else 0
    Zc = min(int(Z), N)
    out = torch.empty((*Y.shape[:-1], Zc), dtype=torch.int32, device=Y.device)
    vals = torch.empty(out.shape, dtype=torch.float32, device=Y.device) if return_values else None
    lib = _lib.load()
    nws = lib.fm_argtopz_workspace(rows, N, int(Z))             # non-zero only for lists longer than FM_MAX_Z
    ws = _ws(nws, Y) if nws else None
    check(lib.fm_argtopz_f32(_p(Y), rows, N, N, int(Z), _p(out), _p(vals), _p(ws), nws, _stream(Y)))
    return (out, vals) if return_values else out


last_build_info = {}


class DeferredBuildStatus:
    """Status word of a fused index build that has not been read back yet (``build_index(..., defer_check=True)``):
    ``unresolved()`` synchronises with the build's stream and says whether rows were left for the unfused build."""

    def __init__(self, status: Optional[torch.Tensor]):
        self.status = status                 # the device status word of fm_build_index_fused; None = unfused
        self._host = None

    def read(self) -> Tuple[int, int]:
        if self._host is None:
            st = [0, 0] if self.status is None else self.status.tolist()
            self._host = (st[0], st[1])
            last_build_info.update(rows_repaired=st[0], rows_unresolved=st[1], repaired_rows=[r for r in st[2:] if r >= 0])
        return self._host

    def unresolved(self) -> int:
        return self.read()[1]


def build_index(A: torch.Tensor, K: torch.Tensor, Z: int, workspace_bytes: int = 8 << 30,
                fused: Optional[bool] = None, return_values: bool = False, defer_check: bool = False):
    """Bucket lists [H,C,min(Z,N)] int32 (memory.py:260-278 on one device); with ``return_values`` also
    the fp32 projections of the listed keys (what an index needs to be extended later).

    ``fused=None`` takes the fused build (no Y in memory) where the shape is
    eligible and H * C * N is at least 2^24, and the unfused one otherwise; both give identical lists.  The
    fused build reports through a two-int status on the device whether any row could not be
    resolved there, in which case the unfused build runs instead.  Reading that word is the only
    host synchronisation of the build: with ``defer_check`` it is left out, the lists come back with a
    :class:`DeferredBuildStatus` as last element and the caller decides when to look (rows left
    unresolved, more than 64 whose sampled threshold missed, hold keys ``0..Z-1`` until then: valid
    indices, not the right ones)."""
    _dev(A, K)
    H, C, d = A.shape
    _, N, _ = K.shape
    assert K.shape[0] == H and K.shape[2] == d and A.dtype == K.dtype
    lib = _lib.load()
    out = torch.empty((H, C, min(int(Z), N)), dtype=torch.int32, device=A.device)
    vals = torch.empty(out.shape, dtype=torch.float32, device=A.device) if return_values else None

    def done(st=None):
        res = (out, vals) if return_values else (out,)
        if defer_check:
            res = res + (DeferredBuildStatus(st),)
        return res if len(res) > 1 else res[0]

    fws = lib.fm_build_index_fused_workspace(H, C, N, d, int(Z), _dt(A)) if fused is not False else 0
    if fused and not fws:
        raise ValueError("fused index build: shape not eligible (bf16 / fp16, d=128, N>=16384, 64<=Z<=N/8)")
    if fused is None and H * C * N < (1 << 24):
        fws = 0          # a small build: the fixed cost of the fused form's four phases is more than it saves
    if fws:
        ws = _ws(fws, A)
        status = torch.empty(_lib.FM_FUSED_STATUS_INTS, dtype=torch.int32, device=A.device)
        check(lib.fm_build_index_fused(_p(A), _p(K), _p(out), _p(vals), H, C, N, d, int(Z), _dt(A), _p(ws), ws.numel(),
                                       _p(status), _stream(A)))
        del ws
        last_build_info.update(path="fused", rows_repaired=None, rows_unresolved=None)
        if defer_check:
            return done(status)
        st_host = status.tolist()                       # the one read-back of a build
        repaired, unresolved = st_host[0], st_host[1]
        last_build_info.update(rows_repaired=repaired, rows_unresolved=unresolved,
                               repaired_rows=[r for r in st_host[2:] if r >= 0])
        if unresolved == 0:
            return done()
    build_index_unfused_(A, K, Z, out, vals, workspace_bytes)
    return done()


def build_index_unfused_(A, K, Z: int, out: torch.Tensor, vals: Optional[torch.Tensor], workspace_bytes: int = 8 << 30):
    """The unfused build (projection rows into a workspace, arg-top-Z from there) into ``out`` / ``vals``."""
    H, C, d = A.shape
    N = K.shape[1]
    lib = _lib.load()
    last_build_info.update(path="unfused")
    full = lib.fm_build_index_workspace(H, C, N, d, int(Z), H * C)     # every row at once if the budget allows
    one = lib.fm_build_index_workspace(H, C, N, d, int(Z), 1)
    ws = _ws(max(one, min(full, int(workspace_bytes))), A)
    check(lib.fm_build_index(_p(A), _p(K), _p(out), _p(vals), H, C, N, d, int(Z), _dt(A), _p(ws), ws.numel(),
                             _stream(A)))


def index_append(A: torch.Tensor, K_new: torch.Tensor, n_old: int, idx: torch.Tensor, val: torch.Tensor, Z: int,
                 inplace: bool = False):
    """Merge M new keys (global indices n_old..n_old+M-1) into bucket lists ``idx`` / ``val``
    [H,C,min(Z,n_old)]: the lists a rebuild over all keys would give (memory.py:252-278 rebuilds).
    Returns ``(idx, val)`` [H,C,min(Z,n_old+M)], or ``None`` when a bucket took more new keys than the
    merge buffers hold (rebuild then).  ``inplace`` (full lists only) updates ``idx`` / ``val`` themselves
    and touches only the buckets that take a new key; after ``None`` they are damaged."""
    _dev(A, K_new, idx, val)
    H, C, d = A.shape
    _, M, _ = K_new.shape
    assert K_new.shape[0] == H and K_new.shape[2] == d and A.dtype == K_new.dtype
    L_in = min(int(Z), int(n_old))
    assert idx.shape == (H, C, L_in) and val.shape == (H, C, L_in)
    assert idx.dtype == torch.int32 and val.dtype == torch.float32 and idx.is_contiguous() and val.is_contiguous()
    L_out = min(int(Z), int(n_old) + M)
    lib = _lib.load()
    if inplace:
        assert L_in == L_out, "in place needs full lists (n_old >= Z)"
        idx2, val2 = idx, val
    else:
        idx2 = torch.empty((H, C, L_out), dtype=torch.int32, device=A.device)
        val2 = torch.empty((H, C, L_out), dtype=torch.float32, device=A.device)
    ws = _ws(lib.fm_index_append_workspace(H, C, M), A)
    status = torch.empty(1, dtype=torch.int32, device=A.device)
    check(lib.fm_index_append(_p(A), _p(K_new.contiguous()), int(n_old), M, _p(idx), _p(val), _p(idx2), _p(val2), H, C,
                              int(Z), d, _dt(A), _p(ws), ws.numel(), _p(status), _stream(A)))
    if int(status.item()) != 0:
        return None
    return idx2, val2


# --------------------------------------------------------------------- a3
def qhash(A: torch.Tensor, q: torch.Tensor, return_scores: bool = False):
    """h_q = argmax_c A[h,c,:].q, first maximum wins (memory.py:281-283).  q [H,Sq,d]."""
    _dev(A, q)
    H, C, d = A.shape
    H2, Sq, d2 = q.shape
    assert H == H2 and d == d2 and A.dtype == q.dtype
    out = torch.empty((H, Sq), dtype=torch.int32, device=q.device)
    scores = torch.empty((H, Sq, C), dtype=torch.float32, device=q.device) if return_scores else None
    check(_lib.load().fm_qhash(_p(A), _p(q), _p(out), _p(scores), H, C, Sq, d, _dt(A), _stream(q)))
    return (out, scores) if return_scores else out


# --------------------------------------------------------------------- a4
def window_filter(k_idx: torch.Tensor, lo: int, hi: int):
    """Keep bucket entries in [lo,hi), re-base by -lo (memory.py:128-142).

    k_idx [H,C,Z] int32 -> (flat int32 buffer of H*C*Z slots of which the first
    sum(cnt) are valid, cnt [H,C] int32, off [H,C] int64)."""
    _dev(k_idx)
    assert k_idx.dtype == torch.int32 and k_idx.dim() == 3
    H, C, Z = k_idx.shape
    flat = torch.empty(H * C * Z, dtype=torch.int32, device=k_idx.device)
    cnt = torch.empty((H, C), dtype=torch.int32, device=k_idx.device)
    off = torch.empty((H, C), dtype=torch.int64, device=k_idx.device)
    check(_lib.load().fm_window_filter(_p(k_idx), H * C, Z, int(lo), int(hi), _p(flat), _p(cnt), _p(off),
                                       None, 0, _stream(k_idx)))
    return flat, cnt, off


def bucket_offsets(cnt: torch.Tensor) -> torch.Tensor:
    """Exclusive prefix sum over the flattened counts (triton_kernel.py:86-88)."""
    _dev(cnt)
    assert cnt.dtype == torch.int32
    off = torch.empty(cnt.shape, dtype=torch.int64, device=cnt.device)
    check(_lib.load().fm_bucket_offsets(_p(cnt), cnt.numel(), _p(off), _stream(cnt)))
    return off


# --------------------------------------------------------------------- a5
class QueryGroups(NamedTuple):
    q_perm: torch.Tensor      # [H,Sq] int32
    bin_count: torch.Tensor   # [H,C]  int32
    bin_off: torch.Tensor     # [H,C]  int32
    items: torch.Tensor       # [max_items,4] int32
    n_items: torch.Tensor     # [1] int32
    max_items: int


def group_queries(q_hash: torch.Tensor, C: int) -> QueryGroups:
    """Stable grouping of queries by (row, bucket) on the device (triton_kernel.py:75-88)."""
    _dev(q_hash)
    assert q_hash.dtype == torch.int32 and q_hash.dim() == 2
    H, Sq = q_hash.shape
    lib = _lib.load()
    dev = q_hash.device
    max_items = lib.fm_group_max_items(H, C, Sq)
    q_perm = torch.empty((H, Sq), dtype=torch.int32, device=dev)
    bin_count = torch.empty((H, C), dtype=torch.int32, device=dev)
    bin_off = torch.empty((H, C), dtype=torch.int32, device=dev)
    items = torch.empty((max_items, 4), dtype=torch.int32, device=dev)
    n_items = torch.empty(1, dtype=torch.int32, device=dev)
    ws = _ws(lib.fm_group_queries_workspace(H, C, Sq), q_hash)
    check(lib.fm_group_queries(_p(q_hash), H, C, Sq, _p(q_perm), _p(bin_count), _p(bin_off), _p(items),
                               _p(n_items), max_items, _p(ws), ws.numel(), _stream(q_hash)))
    return QueryGroups(q_perm, bin_count, bin_off, items, n_items, max_items)


# --------------------------------------------------------------------- a6-a8
def hash_attn_fwd(q, k, v, k_idx, bucket_off, bucket_cnt, groups: QueryGroups, sm_scale: float):
    """Bucket-gathered attention (triton_kernel.py:137-272).  q [H,Sq,d], k,v [H,N,d].
    Returns out [H,Sq,d] (q dtype) and lse [H,Sq] fp32 natural log, original query order."""
    _dev(q, k, v, k_idx, bucket_off, bucket_cnt)
    H, Sq, d = q.shape
    _, N, _ = k.shape
    C = bucket_cnt.shape[-1]
    assert k.shape == v.shape and k.shape[0] == H and k.shape[2] == d
    assert q.dtype == k.dtype == v.dtype
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and bucket_off.dtype == torch.int64
    out = torch.empty_like(q)
    lse = torch.empty((H, Sq), dtype=torch.float32, device=q.device)
    lib = _lib.load()
    ws = torch.empty(int(lib.fm_hash_attn_fwd_workspace(groups.max_items)), dtype=torch.uint8, device=q.device)
    check(lib.fm_hash_attn_fwd_ws(_p(q), _p(k), _p(v), _pl(k_idx), _p(bucket_off), _p(bucket_cnt),
                                  _p(groups.q_perm), _p(groups.items), _p(groups.n_items),
                                  groups.max_items, _p(out), _p(lse), H, Sq, N, d, C,
                                  float(sm_scale), _dt(q), _p(ws), ws.numel(), _stream(q)))
    return out, lse


def lists_key_order(k_idx, bucket_off, bucket_cnt, N: int, return_unsorted: bool = False):
    """The flat lists ``k_idx`` with every bucket's entries in ascending key order (same ``bucket_off`` /
    ``bucket_cnt``): the order in which :func:`hash_attn_fwd` and the backward read K and V fastest when many
    queries are served (their results do not depend on the order beyond fp32 rounding; the kernel of
    triton_kernel.py:230-272 takes the lists as stored).  A list that repeats a key or names one outside
    ``[0, N)`` is copied unchanged; with ``return_unsorted`` also the device counter ``[1]`` of such lists."""
    _dev(k_idx, bucket_off, bucket_cnt)
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and bucket_off.dtype == torch.int64
    assert k_idx.is_contiguous() and bucket_off.is_contiguous() and bucket_cnt.is_contiguous()
    assert bucket_off.numel() == bucket_cnt.numel()
    out = torch.empty_like(k_idx)
    n_uns = torch.empty(1, dtype=torch.int32, device=k_idx.device) if return_unsorted else None
    check(_lib.load().fm_lists_key_order(_pl(k_idx), _p(bucket_off), _p(bucket_cnt), bucket_cnt.numel(), int(N),
                                         _p(out), _p(n_uns) if n_uns is not None else None, _stream(k_idx)))
    return (out, n_uns) if return_unsorted else out


def hash_attn_bwd(q, k, v, k_idx, bucket_off, bucket_cnt, groups: QueryGroups, out, lse, dout, sm_scale: float,
                  dk: Optional[torch.Tensor] = None, dv: Optional[torch.Tensor] = None,
                  dlse: Optional[torch.Tensor] = None):
    """Backward of :func:`hash_attn_fwd` (memory.py:166-206 on the gathered pairs).  ``out`` / ``lse`` are
    the forward's result or the merged one; ``dout [H,Sq,d]``.  Returns ``dq`` (dtype of q) and the fp32
    ``dk``, ``dv [H,N,d]``; when ``dk`` / ``dv`` are given the gradients are added into them.  ``dlse [H,Sq]``
    fp32 (optional) is the gradient w.r.t. the returned log-sum-exp."""
    _dev(q, k, v, k_idx, bucket_off, bucket_cnt, out, lse, dout)
    dlse = _check_dlse(dlse, lse)
    H, Sq, d = q.shape
    _, N, _ = k.shape
    C = bucket_cnt.shape[-1]
    assert k.shape == v.shape and out.shape == q.shape and dout.shape == q.shape and lse.shape == (H, Sq)
    assert q.dtype == k.dtype == v.dtype == out.dtype == dout.dtype and lse.dtype == torch.float32
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and bucket_off.dtype == torch.int64
    if d == 64 and q.dtype in (torch.bfloat16, torch.float16) and not generic_kernels_forced():
        # The MFMA backward is built for d = 128; at d = 64 the generic kernel (an atomic add per query, key and
        # dimension) is twenty times slower than that kernel on rows padded with zeros, which add nothing to
        # any dot product: the same sums, on copies twice the size.
        pad = lambda t: torch.nn.functional.pad(t, (0, 64))
        dq, dk2, dv2 = hash_attn_bwd(pad(q), pad(k), pad(v), k_idx, bucket_off, bucket_cnt, groups, pad(out), lse,
                                     pad(dout), sm_scale, dlse=dlse)
        dk2, dv2 = dk2[..., :64], dv2[..., :64]
        if dk is not None:
            dk2 = dk.add_(dk2)
        if dv is not None:
            dv2 = dv.add_(dv2)
        return dq[..., :64].contiguous(), dk2.contiguous(), dv2.contiguous()
    dq = torch.empty_like(q)
    if dk is None:
        dk = torch.zeros((H, N, d), dtype=torch.float32, device=q.device)
    if dv is None:
        dv = torch.zeros((H, N, d), dtype=torch.float32, device=q.device)
    assert dk.dtype == dv.dtype == torch.float32 and dk.shape == dv.shape == (H, N, d)
    check(_lib.load().fm_hash_attn_bwd(_p(q), _p(k), _p(v), _pl(k_idx), _p(bucket_off), _p(bucket_cnt),
                                       _p(groups.q_perm), _p(groups.items), _p(groups.n_items), groups.max_items,
                                       _p(out), _p(lse), _p(dout), _p(dlse), _p(dq), _p(dk), _p(dv), H, Sq, N, d, C,
                                       float(sm_scale), _dt(q), _stream(q)))
    return dq, dk, dv


def _check_dlse(dlse: Optional[torch.Tensor], lse: torch.Tensor) -> Optional[torch.Tensor]:
    if dlse is None:
        return None
    assert dlse.shape == lse.shape and dlse.is_cuda
    return dlse.to(torch.float32).contiguous()


last_inverse_info = {}


class InverseIndex(NamedTuple):
    """For every key the flat list positions that name it (see ``fm_inverse_index``); depends on the bucket
    lists only, so it can be kept with them."""
    key_off: torch.Tensor      # [H*N + 1] int32
    inv_pos: torch.Tensor      # [T] int32
    row_pos: Tuple[int, ...]   # H + 1 host integers: flat list position where each row's lists begin


def inverse_index(k_idx: torch.Tensor, bucket_off: torch.Tensor, bucket_cnt: torch.Tensor, N: int) -> InverseIndex:
    """Inverse of the flat bucket lists ``k_idx`` (row-major (row, bucket) order, ``bucket_off`` / ``bucket_cnt``
    [H,C]) over keys 0..N-1 of every row.  ``k_idx`` may be longer than the lists (only
    the first ``sum(bucket_cnt)`` entries are read).  Synchronises (the rows' list boundaries and the count of entries out of key order are read back)."""
    _dev(k_idx, bucket_off, bucket_cnt)
    H, C = bucket_cnt.shape
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and bucket_off.dtype == torch.int64
    # the listed entries are the first T of k_idx; a buffer from the window filter is longer (it has room
    # for every entry of the unfiltered lists) and its tail is not initialised
    lib = _lib.load()
    dev = k_idx.device
    starts = bucket_off[:, 0].cpu().tolist()
    T = int(bucket_off[-1, -1]) + int(bucket_cnt[-1, -1])
    assert 0 <= T <= k_idx.numel(), "k_idx is shorter than the lists bucket_off / bucket_cnt describe"
    key_off = torch.empty(H * N + 1, dtype=torch.int32, device=dev)
    inv_pos = torch.empty(T, dtype=torch.int32, device=dev)
    path = "none"
    if not T:
        key_off.zero_()
    elif C > 65535:
        ws = _ws(lib.fm_inverse_index_workspace(T, H, N), k_idx)
        check(lib.fm_inverse_index(_p(k_idx), _p(bucket_off), _p(bucket_cnt), H, C, int(N), T, _p(key_off),
                                   _p(inv_pos), _p(ws), ws.numel(), _stream(k_idx)))
        path = "sort"
    else:
        # lists in strictly ascending key order (what Memory keeps for its attention) are inverted by a
        # transposition, which also counts the entries out of order; any other lists by a sort
        n_bad = torch.empty(1, dtype=torch.int32, device=dev)
        ws = _ws(lib.fm_inverse_index_key_order_workspace(H, C, int(N)), k_idx)
        check(lib.fm_inverse_index_key_order(_p(k_idx), _p(bucket_off), _p(bucket_cnt), H, C, int(N), T, _p(key_off),
                                             _p(inv_pos), _p(n_bad), _p(ws), ws.numel(), _stream(k_idx)))
        path = "transposition"
        if int(n_bad.item()):
            del ws
            ws = _ws(lib.fm_inverse_index_workspace(T, H, N), k_idx)
            check(lib.fm_inverse_index(_p(k_idx), _p(bucket_off), _p(bucket_cnt), H, C, int(N), T, _p(key_off),
                                       _p(inv_pos), _p(ws), ws.numel(), _stream(k_idx)))
            path = "sort"
    last_inverse_info.update(path=path)
    row_pos = tuple(starts) + (T,)
    return InverseIndex(key_off, inv_pos, row_pos)


def hash_attn_bwd_staged(q, k, v, k_idx, bucket_off, bucket_cnt, groups: QueryGroups, inv: InverseIndex, out, lse,
                         dout, sm_scale: float, dk: Optional[torch.Tensor] = None,
                         dv: Optional[torch.Tensor] = None, workspace_bytes: int = 24 << 30,
                         dlse: Optional[torch.Tensor] = None):
    """:func:`hash_attn_bwd` without atomics (bf16 or fp16, d = 128): per-bucket bf16 partial rows in a workspace, then a
    sum per key over the list positions that name it (``inv`` from :func:`inverse_index`).  Same results to
    rounding (the partial rows are bf16), in a fixed summation order."""
    _dev(q, k, v, k_idx, bucket_off, bucket_cnt, out, lse, dout)
    dlse = _check_dlse(dlse, lse)
    H, Sq, d = q.shape
    _, N, _ = k.shape
    C = bucket_cnt.shape[-1]
    assert k.shape == v.shape and out.shape == q.shape and dout.shape == q.shape and lse.shape == (H, Sq)
    assert q.dtype == k.dtype == v.dtype == out.dtype == dout.dtype and q.dtype in (torch.bfloat16, torch.float16)
    if d == 64:      # on rows padded with zeros, as in hash_attn_bwd
        pad = lambda t: torch.nn.functional.pad(t, (0, 64))
        dq, dk2, dv2 = hash_attn_bwd_staged(pad(q), pad(k), pad(v), k_idx, bucket_off, bucket_cnt, groups, inv, pad(out),
                                            lse, pad(dout), sm_scale, workspace_bytes=workspace_bytes, dlse=dlse)
        dk2, dv2 = dk2[..., :64], dv2[..., :64]
        if dk is not None:
            dk2 = dk.add_(dk2)
        if dv is not None:
            dv2 = dv.add_(dv2)
        return dq[..., :64].contiguous(), dk2.contiguous(), dv2.contiguous()
    assert d == 128
    assert len(inv.row_pos) == H + 1 and inv.key_off.numel() == H * N + 1
    dq = torch.zeros_like(q)                                  # queries of an empty bucket keep 0
    if dk is None:
        dk = torch.zeros((H, N, d), dtype=torch.float32, device=q.device)
    if dv is None:
        dv = torch.zeros((H, N, d), dtype=torch.float32, device=q.device)
    assert dk.dtype == dv.dtype == torch.float32 and dk.shape == dv.shape == (H, N, d)
    lib = _lib.load()
    longest = max(inv.row_pos[h + 1] - inv.row_pos[h] for h in range(H))
    total = inv.row_pos[H] - inv.row_pos[0]
    need_all = lib.fm_hash_attn_bwd_staged_workspace(total)
    ws = _ws(min(need_all, max(int(workspace_bytes), lib.fm_hash_attn_bwd_staged_workspace(longest))), q)
    row_pos = (ctypes.c_int64 * (H + 1))(*inv.row_pos)
    check(lib.fm_hash_attn_bwd_staged(_p(q), _p(k), _p(v), _pl(k_idx), _p(bucket_off), _p(bucket_cnt),
                                      _p(groups.q_perm), _p(groups.bin_off), _p(groups.bin_count), _p(out), _p(lse),
                                      _p(dout), _p(dlse), _p(inv.key_off), _p(inv.inv_pos), _p(dq), _p(dk),
                                      _p(dv), H, Sq, N, d, C, ctypes.cast(row_pos, ctypes.c_void_p), float(sm_scale),
                                      _dt(q), _p(ws), ws.numel(), _stream(q)))
    return dq, dk, dv


def attention_hash_varlen_i32(q, k, v, k_idx, bucket_cnt, q_hash, sm_scale: float):
    """The reference operator in one C call (triton_kernel.py:51-119) on int32 index tensors."""
    _dev(q, k, v, k_idx, bucket_cnt, q_hash)
    H, Sq, d = q.shape
    _, N, _ = k.shape
    C = bucket_cnt.shape[-1]
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and q_hash.dtype == torch.int32
    lib = _lib.load()
    ws = _ws(lib.fm_attention_hash_varlen_workspace(H, C, Sq), q)
    out = torch.empty_like(q)
    lse = torch.empty((H, Sq), dtype=torch.float32, device=q.device)
    check(lib.fm_attention_hash_varlen(_p(q), _p(k), _p(v), _pl(k_idx), _p(bucket_cnt), _p(q_hash), _p(out),
                                       _p(lse), H, Sq, N, d, C, float(sm_scale), _dt(q), _p(ws),
                                       ws.numel(), _stream(q)))
    return out, lse


def attention_hash_varlen_static_(q, k, v, k_idx, bucket_cnt, q_hash, sm_scale: float, out: torch.Tensor,
                                  lse: torch.Tensor):
    """:func:`attention_hash_varlen_i32` into caller-provided ``out`` / ``lse`` with no allocation at all:
    the grouping scratch is the library's own static device array (``fm_attention_hash_varlen_static``;
    extents beyond ``FM_STATIC_SCRATCH_BYTES`` raise).  Calls on one GPU share that array, so they must
    not overlap."""
    _dev(q, k, v, k_idx, bucket_cnt, q_hash, out, lse)
    H, Sq, d = q.shape
    _, N, _ = k.shape
    C = bucket_cnt.shape[-1]
    assert k_idx.dtype == torch.int32 and bucket_cnt.dtype == torch.int32 and q_hash.dtype == torch.int32
    assert out.shape == q.shape and out.dtype == q.dtype and lse.shape == (H, Sq) and lse.dtype == torch.float32
    check(_lib.load().fm_attention_hash_varlen_static(_p(q), _p(k), _p(v), _pl(k_idx), _p(bucket_cnt), _p(q_hash),
                                                      _p(out), _p(lse), H, Sq, N, d, C, float(sm_scale), _dt(q),
                                                      _stream(q)))
    return out, lse


def decode_hash_attn(q, A_all, K_all, V_all, idx_all, desc, sm_scale: float, return_scores: bool = False):
    """Hash + gathered attention for a decode batch of rows with different memories.
    q [rows,G,d]; A_all [sum C,d]; K_all,V_all [sum N,d]; idx_all flat int32; desc [rows,5] int64
    viewed as fm_rowdesc (a_off, k_off, idx_off, (n_keys | n_buckets<<32), (bucket_size | q_row1<<32))."""
    _dev(q, A_all, K_all, V_all, idx_all, desc)
    rows, G, d = q.shape
    assert desc.dtype == torch.int64 and desc.shape == (rows, 5) and idx_all.dtype == torch.int32
    if G > 16:      # the kernel takes up to 16 query heads per row: more go through in groups of 16
        parts = [decode_hash_attn(q[:, g0:g0 + 16].contiguous(), A_all, K_all, V_all, idx_all, desc, sm_scale,
                                  return_scores) for g0 in range(0, G, 16)]
        return tuple(torch.cat([p[j] for p in parts], dim=1) for j in range(len(parts[0])))
    out = torch.empty_like(q)
    lse = torch.empty((rows, G), dtype=torch.float32, device=q.device)
    h = torch.empty((rows, G), dtype=torch.int32, device=q.device)
    scores = torch.empty((A_all.shape[0], G), dtype=torch.float32, device=q.device) if return_scores else None
    check(_lib.load().fm_decode_hash_attn(_p(q), _p(A_all), _p(K_all), _p(V_all), _p(idx_all), _p(desc), rows, G, d,
                                          float(sm_scale), _p(out), _p(lse), _p(h), _p(scores), _dt(q),
                                          _stream(q)))
    return (out, lse, h, scores) if return_scores else (out, lse, h)


# --------------------------------------------------------------------- a11
def local_attn_fwd(q, k, v, sm_scale: float, causal: bool = True):
    """Dense GQA attention with LSE (call site memory.py:302).  q [H*G,S,d], k,v [H,L,d]."""
    _dev(q, k, v)
    HG, S, d = q.shape
    H, L, _ = k.shape
    assert HG % H == 0 and k.shape == v.shape and k.shape[2] == d and q.dtype == k.dtype == v.dtype
    out = torch.empty_like(q)
    lse = torch.empty((HG, S), dtype=torch.float32, device=q.device)
    check(_lib.load().fm_local_attn_fwd(_p(q), _p(k), _p(v), _p(out), _p(lse), H, HG // H, S, L, d,
                                        float(sm_scale), int(bool(causal)), _dt(q), _stream(q)))
    return out, lse


# --------------------------------------------------------------------- a10
def lse_merge_(out: torch.Tensor, lse: torch.Tensor, block_out: torch.Tensor, block_lse: torch.Tensor):
    """In-place merge of (block_out, block_lse) into the fp32 running pair (memory.py:54-71)."""
    _dev(out, lse, block_out, block_lse)
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and block_lse.dtype == torch.float32
    d = out.shape[-1]
    Q = out.numel() // d
    assert lse.numel() == Q and block_lse.numel() == Q and block_out.numel() == out.numel()
    check(_lib.load().fm_lse_merge(_p(out), _p(lse), _p(block_out), _p(block_lse), Q, d, _dt(block_out),
                                   _stream(out)))
    return out, lse


# --------------------------------------------------------------------- a12/a13
def l2_normalize(X: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    _dev(X)
    d = X.shape[-1]
    Xn = torch.empty_like(X)
    check(_lib.load().fm_l2_normalize(_p(X), _p(Xn), X.numel() // d, d, float(eps), _dt(X), _stream(X)))
    return Xn


def topk_mean(Xn: torch.Tensor, top_idx: torch.Tensor, H: int, G: int, normalize: bool = True) -> torch.Tensor:
    """Xn [H*G,N,d] unit rows, top_idx [C,H*G,k] int32 -> A [C,H,d] (memory.py:224-229, 258)."""
    _dev(Xn, top_idx)
    HG, N, d = Xn.shape
    C, HG2, k = top_idx.shape
    assert HG == HG2 == H * G and top_idx.dtype == torch.int32
    A = torch.empty((C, H, d), dtype=Xn.dtype, device=Xn.device)
    check(_lib.load().fm_topk_mean(_p(Xn), _p(top_idx), _p(A), C, H, G, N, k, d, int(normalize), _dt(Xn),
                                   _stream(Xn)))
    return A


def segment_mean(X: torch.Tensor, groups: QueryGroups, prev: torch.Tensor,
                 normalize_rows: Optional[float] = None) -> torch.Tensor:
    """Spherical K-means update: X [H,N,d] unit rows grouped by label -> centroids [H,C,d].  With
    ``normalize_rows=eps`` the rows may have any length: a member contributes ``x / max(|x|, eps)``, so
    no normalised copy of X is needed."""
    _dev(X, prev)
    H, N, d = X.shape
    _, C, _ = prev.shape
    assert prev.dtype == X.dtype
    out = torch.empty_like(prev)
    lib = _lib.load()
    if normalize_rows is None:
        check(lib.fm_segment_mean(_p(X), _p(groups.q_perm), _p(groups.bin_off), _p(groups.bin_count),
                                  _p(prev), _p(out), H, C, N, d, _dt(X), _stream(X)))
    else:
        check(lib.fm_segment_mean_directions(_p(X), _p(groups.q_perm), _p(groups.bin_off), _p(groups.bin_count),
                                             _p(prev), _p(out), H, C, N, d, float(normalize_rows), _dt(X),
                                             _stream(X)))
    return out


def segment_sum(X: torch.Tensor, perm: torch.Tensor, seg_off: torch.Tensor, seg_cnt: torch.Tensor) -> torch.Tensor:
    """fp32 sums of the rows of X [H,N,d] listed per segment: perm int32 row indices (flat, per h), seg_off /
    seg_cnt [H,C] int32 -> [H,C,d] fp32 (the segmented form of scatter_add_, memory.py:449-450)."""
    _dev(X, perm, seg_off, seg_cnt)
    H, N, d = X.shape
    C = seg_cnt.shape[-1]
    assert perm.dtype == seg_off.dtype == seg_cnt.dtype == torch.int32
    out = torch.empty((H, C, d), dtype=torch.float32, device=X.device)
    check(_lib.load().fm_segment_sum(_p(X), _p(perm), _p(seg_off), _p(seg_cnt), _p(out), H, C, N, d, _dt(X),
                                     _stream(X)))
    return out


def _debug_lib():
    """The library, for a diagnostic switch: those take effect only in a process started with
    FASTMEM_DEBUG_HOOKS=1 (the library reads it at its first call), so that no caller of a serving process can
    reroute another caller's kernels; a switch flipped anywhere else would silently do nothing, hence the error."""
    lib = _lib.load()
    if not lib.fm_debug_hooks_enabled():
        raise RuntimeError("libfastmem's diagnostic switches are off in this process: set FASTMEM_DEBUG_HOOKS=1 in "
                           "the environment before the library is first called")
    return lib


def argtopz_exact_only(on: bool) -> None:
    """Diagnostic switch: dense arg-top-Z by exact radix passes only (no sampled one-pass form)."""
    _debug_lib().fm_debug_argtopz_exact_only(int(on))


_generic_forced = False


def force_generic_kernels(on: bool) -> None:
    """Diagnostic switch: route attention through the generic kernels."""
    global _generic_forced
    _generic_forced = bool(on)
    _debug_lib().fm_debug_force_generic(int(on))


def generic_kernels_forced() -> bool:
    return _generic_forced


def fused_filter_kernel_name(H: int, C: int, N: int, d: int, Z: int, dtype: torch.dtype):
    """Name of the filter kernel the fused index build launches for these extents (None: shape not taken)."""
    name = _lib.load().fm_build_index_fused_kernel(H, C, N, d, Z, _DT[dtype])
    return name.decode() if name else None


def hash_attn_fwd_kernel_name(H: int, Sq: int, N: int, d: int, C: int, dtype: torch.dtype) -> str:
    """Name of the kernel :func:`hash_attn_fwd` launches for these extents."""
    return _lib.load().fm_hash_attn_fwd_kernel(H, Sq, N, d, C, _DT[dtype]).decode()


def local_attn_fwd_kernel_name(G: int, S: int, L: int, d: int, dtype: torch.dtype) -> str:
    """Name of the kernel :func:`local_attn_fwd` launches for these extents."""
    return _lib.load().fm_local_attn_fwd_kernel(G, S, L, d, _DT[dtype]).decode()


def wave_pace_state(N: int, C: int, Sq: int, k_idx: torch.Tensor, row: int) -> dict:
    """Where the schedule of the paced per-row launches of ``hash_attn_wave_kernel`` stands for one row of a
    memory (diagnostic; synchronises): mode 0 measuring / 1 paced / 2 given up for a while, and, in 100 MHz ticks
    per key, the next launch's schedule, the fastest schedule kept in the current search, the mean of the launches
    on the held schedule, the unpaced launch, the last launch and its schedule."""
    import ctypes
    out = (ctypes.c_float * 8)()
    check(_lib.load().fm_debug_wave_pace_state(N, C, Sq, _p(k_idx), row, ctypes.cast(out, ctypes.c_void_p)))
    return {"mode": int(out[0]), "ticks_per_key": out[1], "kept_in_search": out[2], "held_launches": out[3], "unpaced": out[4],
            "hold": int(out[5]), "last_launch": out[6], "last_schedule": out[7]}


def hash_attn_fwd_launches(H: int, Sq: int, N: int, d: int, C: int, dtype: torch.dtype) -> int:
    """Number of launches of that kernel one :func:`hash_attn_fwd` call makes (one per row where a row's K
    and V outgrow the last-level cache)."""
    return int(_lib.load().fm_hash_attn_fwd_launches(H, Sq, N, d, C, _DT[dtype]))


def grouped_forward_kernel(which: Optional[str]) -> None:
    """Diagnostic switch for the bf16 / fp16, d = 128 grouped attention forward: ``"staged"`` always takes the
    kernel that shares a bucket's rows among its waves through LDS, one work item per workgroup, in a single
    launch, ``"staged-per-row"`` the same in one launch per row, ``"staged-pairs"`` the same kernel with two
    work items per workgroup, ``"ring"`` the kernel whose rows go from global memory straight into LDS (three
    items per workgroup) in a single launch, ``"ring-per-row"`` the same in one launch per row, ``"wave"`` the kernel that
    gives every work item a wave of its own in a single launch, ``"wave-per-row"`` the same in one launch per
    row (its sweeps paced against the device's clock), ``"wave-per-row-unpaced"`` that without the pacing, ``"wave-auto"`` the same with the dispatch's own choice between the two, ``"gather"``
    always the kernel that gathers the rows into registers, ``"bwd-register-blocks"`` (backward only) makes the
    two-tile pass of the staged backward load its key blocks into registers instead of through LDS a block
    ahead, ``None`` restores the dispatch (the direct loads
    per row where a row's K and V outgrow the last-level cache, the direct loads from 24 queries per bucket
    on average, else staged unless the launch has few and small work items)."""
    global _generic_forced
    _generic_forced = False
    _debug_lib().fm_debug_force_generic({None: 0, "staged": 2, "gather": 3, "staged-pairs": 4, "ring": 5,
                                         "staged-per-row": 6, "ring-per-row": 7, "bwd-register-blocks": 9,
                                         "wave-auto": 10, "wave": 11, "wave-per-row": 12,
                                         "wave-per-row-unpaced": 13}[which])
