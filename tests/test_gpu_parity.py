"""GPU parity tests: every call goes through the C ABI (libfastmem.so) and is
checked against the CPU oracle on the same seeded inputs.  Integer results
(bucket lists, hashes, grouping) must match bit for bit; attention outputs are
held to atol 2e-2 / rtol 1e-2 for bf16 and 1e-4 for fp32, the fp32 LSE to 1e-3
absolute."""
import math

import numpy as np
import pytest
import torch

from oracle import fm_oracle as O
from tests.util import (assert_attn_close, dev, gen, make_attn_case)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from fast_memory_amd import ops as _ops
    from fast_memory_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return _ops


def sync():
    torch.cuda.synchronize()


# ------------------------------------------------------------------ a1
@pytest.mark.parametrize("dtype,H,C,N,d", [
    (torch.float32, 1, 64, 4096, 64),
    (torch.float32, 2, 5, 130, 16),
    (torch.bfloat16, 2, 256, 1000, 128),
    (torch.bfloat16, 1, 130, 257, 64),
    (torch.bfloat16, 2, 200, 700, 256),     # the MFMA kernel for any head dimension that is a multiple of 16
    (torch.float16, 2, 96, 513, 64),
    (torch.float16, 1, 70, 300, 256),
    (torch.bfloat16, 3, 7, 33, 24),         # d not a multiple of 16: generic kernel
])
def test_project(ops, dtype, H, C, N, d):
    g = gen(100)
    A = torch.randn(H, C, d, generator=g).to(dtype)
    K = torch.randn(H, N, d, generator=g).to(dtype)
    Y = ops.project(*dev(A, K)).cpu()
    ref = O.project(A, K)
    assert Y.shape == ref.shape
    # fp32 accumulation of d products of magnitude ~1: a few ulp of sqrt(d)
    assert torch.allclose(Y, ref, atol=2e-4 * math.sqrt(d), rtol=1e-5), (Y - ref).abs().max()


# ------------------------------------------------------------------ a2
def check_topz(ops, Y, Z):
    got = ops.argtopz(dev(Y), Z).cpu()
    ref = O.argtopz(Y, Z)
    assert got.dtype == torch.int32 and got.shape == ref.shape
    assert torch.equal(got.long(), ref), "bucket lists differ from the stable-sort definition"


def test_argtopz_random_rows(ops):
    g = gen(200)
    check_topz(ops, torch.randn(3, 7, 5000, generator=g), 256)
    check_topz(ops, torch.randn(64, 4096, generator=g), 256)
    check_topz(ops, torch.randn(5, 1023, generator=g) * 1e-3, 1)


def test_argtopz_heavy_ties(ops):
    g = gen(201)
    # bf16-valued scores: thousands of exactly equal values straddle the cut
    Y = torch.randn(6, 20000, generator=g).to(torch.bfloat16).float()
    check_topz(ops, Y, 1024)
    # integer-valued rows and an all-equal row (pure index order)
    Yi = torch.randint(-3, 4, (4, 3000), generator=g).float()
    Yi[1] = 2.0
    check_topz(ops, Yi, 500)


def test_argtopz_special_values(ops):
    g = gen(202)
    Y = torch.randn(4, 2048, generator=g)
    Y[0, 5] = math.inf
    Y[0, 77] = -math.inf
    Y[1, ::3] = 0.0
    Y[1, 1::3] = -0.0
    Y[2] = -Y[2].abs() * 1e-40          # negative denormals
    Y[3, 100:200] = math.inf
    for Z in (1, 64, 700, 2048):
        check_topz(ops, Y, Z)


def test_argtopz_clamps_to_n_and_unaligned_rows(ops):
    g = gen(203)
    Y = torch.randn(3, 333, generator=g)
    check_topz(ops, Y, 1000)                                        # Z > N -> full sort of the row
    check_topz(ops, torch.randn(9, 1021, generator=g), 100)          # rows not 16-byte aligned


def test_argtopz_max_z_long_row(ops):
    g = gen(204)
    Y = torch.randn(2, 300000, generator=g)
    check_topz(ops, Y, 16384)


def test_argtopz_sampled_one_pass_equals_exact_passes(ops):
    """Long rows take the sampled one-pass selection (lists longer than 8192 in the form that collects the
    candidates of the two interleaved halves of a row one after the other); rows the sample misleads, or whose
    candidates crowd into one half, fall back inside the kernel.  Both must give the lists of the exact multi-pass
    selection, bit for bit."""
    g = gen(210)
    N = 131072 + 37                                          # ragged tail, rows not 16-byte aligned after row 0
    Y = torch.randn(12, N, generator=g)
    Y[1] = torch.randn(N, generator=g).round()               # heavy ties: a few dozen distinct values
    Y[2] = 1.0                                               # all equal: the threshold keeps the whole row
    Y[3, ::7] = float("inf")
    Y[4, 5::3] = float("nan")
    Y[5] = torch.where(torch.arange(N) % 16 == 0, Y[5] + 100.0, Y[5])     # the large values sit on the sampled lines' lanes
    Y[6, :N // 2] -= 50.0                                    # all large values in the second half
    Y[7] = torch.arange(N, dtype=torch.float32)              # ascending: the top is the tail, which is never sampled
    Y[8] = -torch.arange(N, dtype=torch.float32)
    Y[9, 1000:1000 + 3000] = 7.0                             # a tie block that straddles the cut
    Yd = dev(Y)
    for Z in (128, 1000, 4096, 8192, 12000, 16384):
        fast, fv = ops.argtopz(Yd, Z, return_values=True)
        ops.argtopz_exact_only(True)
        try:
            exact, ev = ops.argtopz(Yd, Z, return_values=True)
        finally:
            ops.argtopz_exact_only(False)
        assert torch.equal(fast, exact), f"Z={Z}: rows {(fast != exact).any(dim=1).nonzero().flatten().tolist()} differ"
        assert torch.equal(fv.view(torch.int32), ev.view(torch.int32))
        rows = [0, 1, 5, 9]
        assert torch.equal(fast[rows].cpu().long(), O.argtopz(Y[rows], Z))


def test_argtopz_beyond_fm_max_z_needs_its_workspace(ops, lib):
    # lists longer than FM_MAX_Z are sorted in a workspace (tests/test_gpu_limits.py checks the results);
    # without one the call is refused with a status code, before any launch
    Y = torch.zeros(1, 40000, device="cuda")
    out = torch.empty(1, 20000, dtype=torch.int32, device="cuda")
    assert lib.fm_argtopz_workspace(1, 40000, 20000) == 32768 * 8
    assert lib.fm_argtopz_workspace(1, 40000, 16384) == 0
    assert lib.fm_argtopz_f32(Y.data_ptr(), 1, 40000, 40000, 20000, out.data_ptr(), None, None, 0, None) == 3
    assert b"workspace" in lib.fm_last_error()


def test_build_index_matches_project_then_select(ops):
    g = gen(205)
    A = torch.randn(2, 40, 128, generator=g).to(torch.bfloat16)
    K = torch.randn(2, 3000, 128, generator=g).to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    Y = ops.project(Ad, Kd)
    lists = ops.build_index(Ad, Kd, 128, workspace_bytes=3000 * 4 * 7)   # forces several passes
    assert torch.equal(lists, ops.argtopz(Y, 128))
    assert torch.equal(lists.cpu().long(), O.argtopz(Y.cpu(), 128))


# ------------------------------------------------------------------ a3
@pytest.mark.parametrize("dtype,H,C,S,d", [
    (torch.float32, 1, 64, 512, 64),
    (torch.bfloat16, 2, 256, 1000, 128),
    (torch.bfloat16, 2, 300, 77, 64),
    (torch.bfloat16, 2, 150, 333, 256),
    (torch.float16, 1, 90, 200, 64),
    (torch.float16, 2, 257, 129, 256),
    (torch.float32, 3, 9, 40, 16),
])
def test_qhash(ops, dtype, H, C, S, d):
    g = gen(300)
    A = torch.randn(H, C, d, generator=g).to(dtype)
    q = torch.randn(H, S, d, generator=g).to(dtype)
    A[0, C - 1] = A[0, 2]                                            # exact tie: bucket 2 must win
    h, sc = ops.qhash(*dev(A, q), return_scores=True)
    h, sc = h.cpu(), sc.cpu()
    assert torch.equal(h.long(), O.argmax_first(sc)), "hash is not the first argmax of the kernel's scores"
    assert not (h[0] == C - 1).any()
    ref_sc = O.qhash_scores(A, q)
    assert torch.allclose(sc, ref_sc, atol=2e-4 * math.sqrt(d), rtol=1e-5)
    ref_h = O.argmax_first(ref_sc)
    diff = h.long() != ref_h
    if diff.any():                                                   # only near-ties may differ
        top2 = torch.topk(ref_sc, 2, dim=-1)[0]
        assert ((top2[..., 0] - top2[..., 1])[diff] < 1e-3).all()
    assert torch.equal(ops.qhash(*dev(A, q)).cpu(), h)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("C", [1, 5, 33, 64, 65, 128, 129, 192, 200, 320, 2051])
def test_qhash_streaming_kernel_tile_counts(ops, dtype, C):
    """The streaming hash kernel (d = 128, no scores written) pipelines 64-row tiles of A through two
    accumulator sets: one, two, three (odd) and many tiles, ragged last tiles, the maximum in the first and in
    the last row, and equal rows in different tiles (the first must win)."""
    g = gen(310 + C)
    H, S = 2, 700
    A = torch.randn(H, C, 128, generator=g).to(dtype)
    q = torch.randn(H, S, 128, generator=g).to(dtype)
    if C > 1:
        A[0, C - 1] = A[0, 0]                                        # equal rows, as far apart as they get
        A[1, C - 1] = 4 * q[1, 0]                                    # query 0 of row 1: the last bucket by far
        if C > 70:
            A[0, 70] = A[0, 37]                                      # equal rows in neighbouring tiles
    h, sc = ops.qhash(*dev(A, q), return_scores=True)
    hs = ops.qhash(*dev(A, q))                                       # the streaming kernel
    assert torch.equal(hs.cpu().long(), O.argmax_first(sc.cpu())), "hash is not the first argmax of the scores"
    assert torch.equal(hs, h)
    if C > 1:
        assert not (hs[0] == C - 1).any()
        assert int(hs[1, 0]) == C - 1
        if C > 70:
            assert not (hs[0] == 70).any()


def test_probe_kernels_run_and_write_nothing(ops):
    """The kernels of known size that the benchmark times for scale (a read stream, an MFMA stream)."""
    from fast_memory_amd import _lib
    lib = _lib.load()
    src = torch.ones(1 << 20, dtype=torch.uint8, device="cuda")
    operands = torch.randn(5120, generator=gen(320)).to(torch.bfloat16).cuda()
    sink = torch.zeros(2, dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(lib.fm_debug_read(src.data_ptr(), src.numel(), sink.data_ptr(), st))
    _lib.check(lib.fm_debug_mfma(operands.data_ptr(), operands.numel(), 3, sink.data_ptr(), st))
    _lib.check(lib.fm_debug_mfma(operands.data_ptr(), operands.numel(), 0, sink.data_ptr(), st))
    # the gather of 256-byte rows: a region every L2 holds (read 2^17 / rows times per sweep), one a sweep
    # covers exactly, and sizes it does not take
    big = torch.ones(32 << 20, dtype=torch.uint8, device="cuda")
    _lib.check(lib.fm_debug_gather(src.data_ptr(), src.numel(), 2, sink.data_ptr(), st))
    _lib.check(lib.fm_debug_gather(big.data_ptr(), big.numel(), 2, sink.data_ptr(), st))
    _lib.check(lib.fm_debug_gather(big.data_ptr(), big.numel(), 0, sink.data_ptr(), st))
    for bad in (256 * 1000, 256 * 512, (1 << 20) + 128):
        assert lib.fm_debug_gather(big.data_ptr(), bad, 1, sink.data_ptr(), st) != 0
    sync()
    assert sink.tolist() == [0.0, 0.0]


# ------------------------------------------------------------------ a4/a5/a16
@pytest.mark.parametrize("H,S,C", [(1, 24, 8), (3, 1000, 17), (8, 8160, 512), (2, 300, 2048)])
def test_group_queries(ops, H, S, C):
    qh = torch.randint(0, C, (H, S), generator=gen(400))
    if S > 100:
        qh[0, : S // 2] = 3                                          # a heavy bucket spanning several tiles
    G = ops.group_queries(dev(qh.int()), C)
    sync()
    perm, gb, gc, go = O.group_queries(qh, C)
    assert torch.equal(G.q_perm.cpu().long(), perm)
    assert torch.equal(G.bin_count.cpu().long(), O.bin_counts(qh, C))
    flat_cnt = G.bin_count.cpu().long().reshape(-1)
    assert torch.equal(G.bin_off.cpu().long().reshape(-1), torch.cumsum(flat_cnt, 0) - flat_cnt)
    n = int(G.n_items.item())
    items = G.items[:n].cpu().long()
    # items tile the groups in (row, bucket) order, at most 64 queries each
    exp = []
    for z, cnt, off in zip(gb.tolist(), gc.tolist(), go.tolist()):
        row = off // S
        for t in range(0, cnt, 64):
            exp.append([row, z, off + t, min(64, cnt - t)])
    assert items.tolist() == exp


@pytest.mark.parametrize("H,S,C", [(2, 300000, 3700), (1, 1100000, 2048), (5, 110000, 4000)])
def test_group_long_rows(ops, H, S, C):
    """Where the table of block counts would take 2^23 words or more the grouping is a stable radix sort instead: same permutation (stable: ascending entry index inside a bucket), bins and items; entries without
    a bucket behind all others, as -(flat index) - 1."""
    g = torch.Generator(device="cuda").manual_seed(402)
    qh = torch.randint(0, C, (H, S), generator=g, device="cuda", dtype=torch.int32)
    qh[0, : S // 3] = 3                                                  # a heavy bucket
    qh[-1, 5::1000] = C + 7                                              # entries without a bucket
    qh[0, 11::777] = -1
    G = ops.group_queries(qh, C)
    valid = (qh >= 0) & (qh < C)
    key = torch.where(valid, qh.long() + torch.arange(H, device="cuda")[:, None] * C, torch.full_like(qh, H * C).long())
    order = torch.sort(key.reshape(-1), stable=True).indices
    n_valid = int(valid.sum())
    exp = torch.where(torch.arange(H * S, device="cuda") < n_valid, order % S, -order - 1).int()
    perm = G.q_perm.reshape(-1)
    assert torch.equal(perm[:n_valid], exp[:n_valid])
    assert torch.equal(torch.sort(perm[n_valid:]).values, torch.sort(exp[n_valid:]).values)
    cnt = torch.bincount(key.reshape(-1), minlength=H * C + 1)[: H * C]
    assert torch.equal(G.bin_count.reshape(-1).long(), cnt)
    assert torch.equal(G.bin_off.reshape(-1).long(), torch.cumsum(cnt, 0) - cnt)
    n = int(G.n_items.item())
    items = G.items[:n].cpu().long()
    tiles = (cnt + 63) // 64
    assert n == int(tiles.sum())
    first = (torch.cumsum(tiles, 0) - tiles).cpu()
    bins = torch.repeat_interleave(torch.arange(H * C), tiles.cpu())
    t_in = torch.arange(n) - first[bins]
    off = (torch.cumsum(cnt, 0) - cnt).cpu()
    exp_items = torch.stack([bins // C, bins % C, off[bins] + 64 * t_in,
                             torch.minimum(torch.full_like(t_in, 64), cnt.cpu()[bins] - 64 * t_in)], 1)
    assert torch.equal(items, exp_items)


def test_bucket_offsets_and_window_filter(ops):
    g = gen(401)
    cnt = torch.randint(0, 50, (7, 300), generator=g).int()
    off = ops.bucket_offsets(dev(cnt)).cpu()
    assert torch.equal(off, O.bucket_offsets(cnt.long()))
    kh = torch.randint(0, 1000, (3, 40, 33), generator=g).int()
    flat, c, o = ops.window_filter(dev(kh), 250, 700)
    rflat, rc = O.window_filter(kh.long(), 250, 700)
    assert torch.equal(c.cpu().long(), rc)
    assert torch.equal(o.cpu(), O.bucket_offsets(rc))
    assert torch.equal(flat[: rflat.numel()].cpu().long(), rflat)


def _ragged_distinct_lists(g, n_lists, N, max_len):
    """Flat ragged lists of distinct keys (each a random subset of [0, N)), offsets, counts."""
    cnt = torch.randint(0, max_len + 1, (n_lists,), generator=g).int()
    cnt[0], cnt[-1] = 0, max_len                       # an empty list and a longest one
    if n_lists > 2:
        cnt[1] = 1
    lists = [torch.randperm(N, generator=g)[: int(c)].int() for c in cnt]
    off = torch.zeros(n_lists, dtype=torch.int64)
    off[1:] = torch.cumsum(cnt.long(), 0)[:-1]
    return lists, off, cnt


@pytest.mark.parametrize("n_lists,N,max_len", [(40, 1000, 700),            # one pass, 256 threads
                                               (9, 262144, 5000),          # the largest single pass of the narrow form
                                               (6, 262145, 70000),         # 512 threads, lists longer than FM_MAX_Z
                                               (4, 600000, 20000),         # 1024 threads, one pass
                                               (5, 3 * (1 << 20) + 77, 3000),   # four passes, ragged last range
                                               (3, 33, 33)])               # every key listed, one bitmap word and a bit
def test_lists_key_order(ops, n_lists, N, max_len):
    g = gen(420 + n_lists)
    max_len = min(max_len, N)
    lists, off, cnt = _ragged_distinct_lists(g, n_lists, N, max_len)
    flat = torch.cat(lists)
    got, n_uns = ops.lists_key_order(dev(flat), dev(off), dev(cnt), N, return_unsorted=True)
    ref = torch.cat([torch.sort(l).values for l in lists])
    assert int(n_uns.item()) == 0
    assert torch.equal(got.cpu(), ref)


def test_lists_key_order_dense_and_thin_stretches(ops):
    """One list with a run of neighbouring keys (more keys in a stretch of the range than a wave stages at once:
    stored lane by lane), a thin spread (staged, stored 64 at a time) and a run that ends on the last key of a
    range whose word count is not a multiple of 4."""
    N = 262144 + 37
    keys = torch.cat([torch.arange(5000, 9000), torch.arange(20000, 260000, 61), torch.arange(N - 70, N)]).int()
    flat = keys[torch.randperm(keys.numel(), generator=gen(3))].contiguous()
    flat = torch.cat([flat, flat[:500].sort().values])        # and a second, short list
    off = torch.tensor([0, keys.numel()], dtype=torch.int64)
    cnt = torch.tensor([keys.numel(), 500], dtype=torch.int32)
    got, n_uns = ops.lists_key_order(dev(flat), dev(off), dev(cnt), N, return_unsorted=True)
    assert int(n_uns.item()) == 0
    assert torch.equal(got.cpu(), torch.cat([keys, flat[keys.numel():]]))


def test_lists_key_order_copies_lists_it_cannot_sort(ops):
    """A list that names a key twice counts it twice in the softmax, and one with an entry outside [0, N) is
    whatever the caller meant: both come back unchanged (and counted), the other lists sorted."""
    g = gen(431)
    N = 5000
    lists, off, cnt = _ragged_distinct_lists(g, 12, N, 900)
    lists[3] = torch.cat([lists[3][:10], lists[3][:10], torch.randperm(N, generator=g)[:50].int()])   # repeats
    lists[7] = torch.cat([torch.tensor([N], dtype=torch.int32), torch.randperm(N, generator=g)[:20].int()])
    lists[9] = torch.cat([torch.randperm(N, generator=g)[:20].int(), torch.tensor([-1], dtype=torch.int32)])
    cnt = torch.tensor([l.numel() for l in lists], dtype=torch.int32)
    off = torch.zeros(12, dtype=torch.int64)
    off[1:] = torch.cumsum(cnt.long(), 0)[:-1]
    flat = torch.cat(lists)
    got, n_uns = ops.lists_key_order(dev(flat), dev(off), dev(cnt), N, return_unsorted=True)
    ref = torch.cat([l if i in (3, 7, 9) else torch.sort(l).values for i, l in enumerate(lists)])
    assert int(n_uns.item()) == 3
    assert torch.equal(got.cpu(), ref)


def test_attention_hash_reorders_lists_by_density(ops):
    """The composite (triton_kernel.py:275-286) hands the attention key-ordered lists between 1 and 96 queries
    per bucket on average: the same result as over the lists as built, and as the oracle's composite."""
    from fast_memory_amd import attention_hash
    from fast_memory_amd.hash_attention import sorts_lists
    assert not sorts_lists(10, 16) and sorts_lists(16, 16) and sorts_lists(95 * 16, 16) and not sorts_lists(96 * 16, 16)
    assert not sorts_lists(131072, 1024) and sorts_lists(32768, 2048)          # the harness shape; the 1M-key one
    g = gen(433)
    B, S, N, C, Z, d = 2, 700, 5000, 20, 300, 128
    q = (torch.randn(B, S, d, generator=g) * 0.5).to(torch.bfloat16)
    k = (torch.randn(B, N, d, generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(B, N, d, generator=g) * 0.5).to(torch.bfloat16)
    A = torch.randn(B, C, d, generator=g).to(torch.bfloat16)
    res = {ko: attention_hash(*dev(q, k, v, A), Z, d ** -0.5, key_order=ko) for ko in (None, True, False)}
    sync()
    assert torch.equal(res[None][0], res[True][0]) and torch.equal(res[None][1], res[True][1])   # 35 per bucket: sorted
    assert (res[True][0].float() - res[False][0].float()).abs().max().item() < 4e-3
    assert (res[True][1] - res[False][1]).abs().max().item() < 1e-4
    lists = O.argtopz(ops.project(*dev(A, k)).cpu(), Z)
    qh = ops.qhash(*dev(A, q)).cpu().long()
    ro, rl = O.hashed_attention_gather(q, k, v, lists.reshape(-1), torch.full((B, C), Z), qh, d ** -0.5)
    assert_attn_close(res[None][0], res[None][1], ro, rl, torch.bfloat16, "attention_hash, key-ordered lists")


def test_memory_attends_over_key_ordered_lists(ops):
    """Memory.attend reads a key-ordered copy of the lists once a call brings a query per bucket: the same
    sets, bucket_idx untouched, the result that of the oracle on the lists as torch.topk orders them; a
    memory built with key_order=False reads bucket_idx itself and agrees to rounding."""
    from fast_memory_amd import Memory
    g = gen(432)
    H, C, N, d, Z, S = 2, 16, 6000, 128, 512, 300
    K = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    V = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
    q = (torch.randn(H, S, d, generator=g) * 0.5).to(torch.bfloat16)
    mem = Memory.build(*dev(K, V, A), Z, keep_values=True)
    plain = Memory.build(*dev(K, V, A), Z, key_order=False)
    idx0 = mem.bucket_idx.clone()
    few = mem.attend(dev(q[:, :8]), d ** -0.5)            # fewer queries than buckets: no copy is made
    assert mem._attn_idx is None
    out, lse = mem.attend(dev(q), d ** -0.5)
    assert mem._attn_idx is not None and torch.equal(mem.bucket_idx, idx0)
    ko = mem._attn_idx.reshape(H, C, Z).cpu()
    assert torch.equal(ko, torch.sort(idx0.cpu(), dim=-1).values)
    qh = mem.hash(dev(q)).cpu().long()
    ro, rl = O.hashed_attention_gather(q, K, V, idx0.cpu().long().reshape(-1), torch.full((H, C), Z), qh, d ** -0.5)
    assert_attn_close(out, lse, ro, rl, torch.bfloat16, "key-ordered lists")
    po, pl = plain.attend(dev(q), d ** -0.5)
    assert plain._attn_idx is None
    assert_attn_close(po, pl, ro, rl, torch.bfloat16, "value-ordered lists")
    assert (out.float() - po.float()).abs().max().item() < 4e-3 and (lse - pl).abs().max().item() < 1e-4
    o8, l8 = mem.attend(dev(q[:, :8]), d ** -0.5)         # the copy exists now and serves small calls too
    assert torch.allclose(o8.float(), few[0].float(), atol=4e-3) and torch.allclose(l8, few[1], atol=1e-4)
    # appending changes the lists: the copy is dropped and made again from the new ones
    mem.append(*dev((torch.randn(H, 40, d, generator=g) * 0.5).to(torch.bfloat16),
                    (torch.randn(H, 40, d, generator=g) * 0.5).to(torch.bfloat16)))
    assert mem._attn_idx is None
    mem.attend(dev(q), d ** -0.5)
    assert torch.equal(mem._attn_idx.reshape(H, C, Z).cpu(), torch.sort(mem.bucket_idx.cpu(), dim=-1).values)


# ------------------------------------------------------------------ a6-a8
def run_varlen(q, k, v, kh, cnt, qh, scale):
    from fast_memory_amd import attention_hash_varlen
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(qd, kd, vd, khd, cntd, qhd, scale)
    sync()
    return out, lse


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_reference_small_shape(dtype):
    # the reference's first test shape (triton_kernel.py:500): B=1,G=1,S=24,N=1024,C=8,Z=16,d=16
    q, k, v, kh, cnt, qh = make_attn_case(20, 1, 24, 1024, 8, 16, 16, dtype)
    out, lse = run_varlen(q, k, v, kh, cnt, qh, 16 ** -0.5)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 16 ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, "ref small")
    ro2, rl2 = O.hashed_attention_dense_masked(q, k, v, kh, cnt, qh, 16 ** -0.5)
    assert_attn_close(out, lse, ro2, rl2, dtype, "ref small (dense-masked)")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_reference_large_shape(dtype):
    # the reference's second test shape (triton_kernel.py:502) with fewer rows so the CPU oracle
    # finishes in seconds: G*S=8160 queries, N=61380, C=512, Z=1024, d=128; the N > 32K window
    # leaves ~20% of the buckets empty
    q, k, v, kh, cnt, qh = make_attn_case(20, 2, 4 * 2040, 1023 * 60, 512, 1024, 128, dtype)
    assert (cnt == 0).any()
    out, lse = run_varlen(q, k, v, kh, cnt, qh, 128 ** -0.5)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 128 ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, "ref large")


@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128), (torch.bfloat16, 64),
                                     (torch.float32, 40), (torch.bfloat16, 256)])
def test_attention_dense_buckets(dtype, d):
    # full-length lists, skewed query groups (one bucket takes half the queries)
    q, k, v, kh, cnt, qh = make_attn_case(21, 2, 700, 4096, 32, 300, d, dtype, window="all", std=1.0)
    qh[0, :350] = 5
    out, lse = run_varlen(q, k, v, kh, cnt, qh, d ** -0.5)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, d ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, f"dense d={d}")


@pytest.mark.parametrize("which", ["staged", "staged-per-row", "staged-pairs", "ring", "ring-per-row", "wave",
                                   "wave-per-row", "gather"])
@pytest.mark.parametrize("case", ["ragged", "full-items", "reference-large", "heavy-bucket"])
def test_attention_grouped_forward_kernels(ops, which, case):
    # the bf16 d=128 forward kernels (rows shared through LDS, one or two work items per workgroup / rows
    # gathered into registers), each forced,
    # against the oracle: ragged lists with a last tile of 1..63 keys and empty buckets; buckets with
    # 1, 15, 16, 17, 63, 64, 65 and 200 queries (several work items, partly filled waves); the
    # reference's large test shape, where ~20% of the buckets are empty; one bucket with 3000 queries
    if case == "ragged":
        q, k, v, kh, cnt, qh = make_attn_case(31, 2, 900, 5000, 24, 333, 128, torch.bfloat16, std=0.7)
    elif case == "full-items":
        q, k, v, kh, cnt, qh = make_attn_case(32, 2, 700, 4096, 40, 300, 128, torch.bfloat16, window="all", std=1.0)
        sizes = [1, 15, 16, 17, 63, 64, 65, 200]
        pos = 0
        for b, n in enumerate(sizes):
            qh[0, pos:pos + n] = b
            pos += n
        qh[0, pos:] = torch.randint(len(sizes), 40, (700 - pos,), generator=gen(33))
    elif case == "heavy-bucket":
        # most of a row's queries in one bucket (dozens of work items of the same bucket), a bucket of exactly
        # 192 and one of 193 queries (the most a workgroup of the direct-load kernel takes, and one more)
        q, k, v, kh, cnt, qh = make_attn_case(34, 2, 3600, 3000, 12, 260, 128, torch.bfloat16, std=0.8)
        qh[0, :3000] = 5
        qh[0, 3000:3192] = 7
        qh[0, 3192:3385] = 2
        qh[0, 3385:] = torch.randint(8, 12, (3600 - 3385,), generator=gen(35))
    else:
        q, k, v, kh, cnt, qh = make_attn_case(20, 1, 4 * 2040, 1023 * 60, 512, 1024, 128, torch.bfloat16)
        assert (cnt == 0).any()
    ops.grouped_forward_kernel(which)
    try:
        out, lse = run_varlen(q, k, v, kh, cnt, qh, 128 ** -0.5)
    finally:
        ops.grouped_forward_kernel(None)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 128 ** -0.5)
    assert_attn_close(out, lse, ro, rl, torch.bfloat16, f"{which} {case}")
    if which.endswith("-per-row"):
        # a launch per row runs the same work items: bit-identical to the single launch (rows without any
        # item, a row whose items end the list, a first item found in the middle of the item list)
        ops.grouped_forward_kernel(which[:-len("-per-row")])
        try:
            o1, l1 = run_varlen(q, k, v, kh, cnt, qh, 128 ** -0.5)
        finally:
            ops.grouped_forward_kernel(None)
        assert torch.equal(out, o1) and torch.equal(lse, l1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("case", ["ragged", "full-items", "reference-large"])
def test_attention_mfma_forward_over_head_dimensions(ops, dtype, d, case):
    """The reference kernel is generic in d_head (triton_kernel.py:141-147; its own test shapes run d = 16 and
    d = 128, triton_kernel.py:500-505).  Head dimensions 64 and 256 take the MFMA kernel whose extents are
    functions of the head dimension -- not the generic one -- and meet the oracle on the cases of the d = 128
    kernels; instantiated for 128 it gives the bits of the kernels built for 128."""
    if case == "ragged":
        q, k, v, kh, cnt, qh = make_attn_case(131, 2, 900, 5000, 24, 333, d, dtype, std=0.7)
    elif case == "full-items":
        q, k, v, kh, cnt, qh = make_attn_case(132, 2, 700, 4096, 40, 300, d, dtype, window="all", std=1.0)
        sizes = [1, 15, 16, 17, 63, 64, 65, 200]
        pos = 0
        for b, n in enumerate(sizes):
            qh[0, pos:pos + n] = b
            pos += n
        qh[0, pos:] = torch.randint(len(sizes), 40, (700 - pos,), generator=gen(133))
    else:
        q, k, v, kh, cnt, qh = make_attn_case(120, 1, 2 * 2040, 1023 * 60, 512, 1024, d, dtype)
        assert (cnt == 0).any()
    H, S, N, C = q.shape[0], q.shape[1], k.shape[1], cnt.shape[1]
    if d != 128:
        name = ops.hash_attn_fwd_kernel_name(H, S, N, d, C, dtype)
        assert name.startswith(f"hash_attn_staged_d_kernel<{d}"), name
        out, lse = run_varlen(q, k, v, kh, cnt, qh, d ** -0.5)
    else:
        from fast_memory_amd import _lib
        _lib.load().fm_debug_force_generic(8)               # the kernel of every head dimension, at 128
        try:
            assert ops.hash_attn_fwd_kernel_name(H, S, N, d, C, dtype).startswith("hash_attn_staged_d_kernel<128")
            out, lse = run_varlen(q, k, v, kh, cnt, qh, d ** -0.5)
        finally:
            ops.grouped_forward_kernel(None)
        ops.grouped_forward_kernel("staged")
        try:
            o1, l1 = run_varlen(q, k, v, kh, cnt, qh, d ** -0.5)
        finally:
            ops.grouped_forward_kernel(None)
        assert torch.equal(out, o1) and torch.equal(lse, l1), "the 128-wide instantiation differs from the staged kernel"
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, d ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, f"d={d} {case}")
    # and against the generic kernel, which defines the numerics of every other shape
    ops.force_generic_kernels(True)
    try:
        og, lg = run_varlen(q, k, v, kh, cnt, qh, d ** -0.5)
    finally:
        ops.force_generic_kernels(False)
    assert_attn_close(out, lse, og.float().cpu(), lg.cpu(), dtype, f"d={d} {case} vs generic")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_with_listed_item_groups(ops, dtype):
    """More than 64 queries per bucket on average: with its workspace the forward lists the groups of three
    items first (fm_hash_attn_fwd_ws), without it a workgroup is started per item and two of three return.  The
    same bits either way, over buckets of 0, 1, 2, 3, 4 and 23 items, the last item of every size, rows with and
    without queries outside every bucket, and more than 1024 items (the listing walks them 1024 at a time)."""
    H, S, N, C, Z, d = 3, 24000, 3000, 60, 150, 128
    q, k, v, kh, cnt, qh = make_attn_case(37, H, S, N, C, Z, d, dtype, std=0.8)
    sizes = [0, 1, 64, 65, 128, 129, 192, 193, 200, 256, 1450, 63]          # queries of buckets 0..11 of row 0
    pos = 0
    for b, n in enumerate(sizes):
        qh[0, pos:pos + n] = b
        pos += n
    qh[0, pos:] = torch.randint(12, C, (S - pos,), generator=gen(38))
    qh[1, ::7] = -1                                                          # in no bucket
    assert ops.hash_attn_fwd_kernel_name(H, S, N, d, C, dtype).startswith("hash_attn_ring_kernel")
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    groups = ops.group_queries(qhd.int(), C)
    assert int(groups.n_items.item()) > 1024
    off = ops.bucket_offsets(cntd.int())
    flat = khd.int().reshape(-1).contiguous()
    from fast_memory_amd import _lib
    lib = _lib.load()
    res = []
    for with_ws in (False, True):
        out = torch.full(q.shape, 7.0, dtype=dtype, device="cuda")
        lse = torch.full((H, S), 7.0, dtype=torch.float32, device="cuda")
        ws = torch.empty(int(lib.fm_hash_attn_fwd_workspace(groups.max_items)) if with_ws else 0, dtype=torch.uint8,
                         device="cuda")
        _lib.check(lib.fm_hash_attn_fwd_ws(
            qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), flat.data_ptr(), off.data_ptr(), cntd.int().contiguous().data_ptr(),
            groups.q_perm.data_ptr(), groups.items.data_ptr(), groups.n_items.data_ptr(), groups.max_items,
            out.data_ptr(), lse.data_ptr(), H, S, N, d, C, float(d ** -0.5), {torch.bfloat16: 1, torch.float16: 2}[dtype],
            ws.data_ptr() if with_ws else None, ws.numel(), torch.cuda.current_stream().cuda_stream))
        sync()
        res.append((out, lse))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    # rows of no bucket: the result of an empty bucket
    assert bool((res[1][1][1, ::7] < -1e30).all()) and bool((res[1][0][1, ::7] == 0).all())
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh.clamp(min=0), d ** -0.5)
    keep = qh >= 0
    assert_attn_close(res[1][0][keep], res[1][1][keep], ro[keep], rl[keep], dtype, "listed groups")


def test_attention_a_launch_per_row_finds_every_rows_items(ops):
    """Eleven rows with very different numbers of work items, among them rows whose queries all carry a hash
    outside [0, C) (no item at all; their rows get the result of an empty bucket): the per-row launches write exactly
    what the single launch writes."""
    H, S, N, C, Z, d = 11, 520, 700, 37, 90, 128
    q, k, v, kh, cnt, qh = make_attn_case(36, H, S, N, C, Z, d, torch.bfloat16, std=0.8)
    qh[3] = -1
    qh[10] = C + 5
    qh[0] = 4                                   # one bucket, nine items
    qh[5, :40] = torch.arange(40) % C           # the rest of row 5 in no bucket
    qh[5, 40:] = -1
    res = []
    for which in ("staged", "staged-per-row", "ring", "ring-per-row", "wave", "wave-per-row"):
        ops.grouped_forward_kernel(which)
        try:
            qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
            groups = ops.group_queries(qhd.int(), C)
            off = ops.bucket_offsets(cntd.int())
            out = torch.full(q.shape, 7.0, dtype=torch.bfloat16, device="cuda")
            lse = torch.full((H, S), 7.0, dtype=torch.float32, device="cuda")
            from fast_memory_amd import _lib
            _lib.check(_lib.load().fm_hash_attn_fwd(
                qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), khd.int().reshape(-1).contiguous().data_ptr(), off.data_ptr(),
                cntd.int().contiguous().data_ptr(), groups.q_perm.data_ptr(), groups.items.data_ptr(),
                groups.n_items.data_ptr(), groups.max_items, out.data_ptr(), lse.data_ptr(), H, S, N, d, C,
                float(d ** -0.5), 1, torch.cuda.current_stream().cuda_stream))
            sync()
            res.append((out.clone(), lse.clone()))
        finally:
            ops.grouped_forward_kernel(None)
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    assert torch.equal(res[2][0], res[3][0]) and torch.equal(res[2][1], res[3][1])
    assert torch.equal(res[4][0], res[5][0]) and torch.equal(res[4][1], res[5][1])
    for _, lse_r in res:
        assert bool((lse_r[3] < -1e30).all()) and bool((lse_r[10] < -1e30).all())         # rows without a bucket
        assert bool((lse_r[5, 40:] < -1e30).all())
        assert bool((lse_r[0] != 7.0).all())


@pytest.mark.parametrize("which", ["staged", "staged-pairs", "ring", "wave", "gather", "generic"])
def test_attention_out_of_range_list_entries_are_clamped(ops, which):
    # the contract of every entry point: key indices outside [0, N) are clamped, never dereferenced
    # (negative -> key 0, >= N -> key N-1); lists here hold such entries in every bucket, and lists
    # shorter than one 64-key tile
    N = 3000
    q, k, v, kh, cnt, qh = make_attn_case(35, 2, 300, N, 12, 150, 128, torch.bfloat16, window="all", std=0.7)
    kh = kh.reshape(2, 12, 150).clone()
    kh[:, :, 3] = -7
    kh[:, :, 77] = N + 1000
    kh[:, :, 149] = 2 ** 31 - 1
    cnt = cnt.clone()
    cnt[0, 5] = 40                                               # a single ragged tile
    cnt[1, 2] = 1
    flat = torch.cat([kh[b, c, : int(cnt[b, c])] for b in range(2) for c in range(12)])
    if which == "generic":
        ops.force_generic_kernels(True)
    else:
        ops.grouped_forward_kernel(which)
    try:
        out, lse = run_varlen(q, k, v, flat, cnt, qh, 128 ** -0.5)
    finally:
        ops.force_generic_kernels(False)
        ops.grouped_forward_kernel(None)
    ro, rl = O.hashed_attention_gather(q, k, v, flat.clamp(0, N - 1), cnt, qh, 128 ** -0.5)
    assert_attn_close(out, lse, ro, rl, torch.bfloat16, f"{which} clamped indices")


def test_attention_special_cases():
    # C=1, Z=N: plain softmax attention; Z=1: out = V[idx]
    g = gen(22)
    B, S, N, d = 2, 9, 200, 64
    q, k, v = (torch.randn(B, n, d, generator=g) for n in (S, N, N))
    kh = torch.stack([torch.randperm(N, generator=g) for _ in range(B)]).reshape(-1)
    out, lse = run_varlen(q, k, v, kh, torch.full((B, 1), N), torch.zeros(B, S, dtype=torch.long), 0.2)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=0.2)
    assert torch.allclose(out.cpu(), ref, atol=1e-4)
    assert torch.allclose(lse.cpu(), torch.logsumexp(q @ k.transpose(1, 2) * 0.2, -1), atol=1e-4)
    kh1 = torch.tensor([7, 2, 5, 1, 0, 3])
    qh1 = torch.randint(0, 3, (B, S), generator=g)
    out, lse = run_varlen(q, k, v, kh1, torch.ones(B, 3, dtype=torch.long), qh1, 0.7)
    for b in range(B):
        sel = kh1[b * 3 + qh1[b]]
        assert torch.allclose(out[b].cpu(), v[b, sel], atol=1e-6)
        assert torch.allclose(lse[b].cpu(), 0.7 * (q[b] * k[b, sel]).sum(-1), atol=1e-4)


def test_attention_reference_lse_rounding_switch():
    from fast_memory_amd import attention_hash_varlen
    q, k, v, kh, cnt, qh = make_attn_case(23, 1, 50, 512, 4, 64, 64, torch.bfloat16, window="all")
    table = kh.reshape(4, 64)
    cnt = torch.tensor([[64, 0, 64, 64]])                            # bucket 1 emptied
    kh = torch.cat([table[0], table[2], table[3]])
    out, lse = attention_hash_varlen(*dev(q, k, v, kh, cnt, qh), 0.125, lse_dtype=None)
    assert lse.dtype == torch.bfloat16
    ro, rl = O.hashed_attention_blocked(q, k, v, kh, cnt, qh, 0.125, ref_lse_rounding=True)
    empty = qh[0] == 1
    assert (lse.cpu()[0][empty] == torch.finfo(torch.bfloat16).min).all()
    # same rounding order as triton_kernel.py:111: bf16(lse2) * ln2 in bf16.  The GPU's fp32 lse2 differs from
    # the oracle's in the last bits (summation order), which moves a bf16 rounding only next to a tie: almost
    # all values are identical and none is further than one bf16 step (2^-7 relative) away
    got, ref = lse.cpu().float()[0][~empty], rl.float()[0][~empty]
    assert (got == ref).float().mean().item() >= 0.95
    assert ((got - ref).abs() <= ref.abs() * 2.0 ** -7 + 1e-6).all()
    # and it is NOT the rounding of the already scaled fp32 value wherever the two orders differ
    ro32, rl32 = O.hashed_attention_blocked(q, k, v, kh, cnt, qh, 0.125)
    other = rl32[0][~empty].to(torch.bfloat16).float()
    differ = other != ref
    assert differ.any(), "case does not separate the two rounding orders"
    assert (got[differ] == ref[differ]).float().mean().item() >= 0.9


# ------------------------------------------------------------------ a10
def test_lse_merge(ops):
    from fast_memory_amd import update_out_and_lse
    g = gen(500)
    oa = torch.randn(3, 40, 128, generator=g)
    ob = torch.randn(3, 40, 128, generator=g).to(torch.bfloat16)
    la = torch.randn(3, 40, generator=g) * 5
    lb = torch.randn(3, 40, generator=g) * 5
    lb[0, :5] = torch.finfo(torch.float32).min                      # empty block: identity
    la[1, :5] = torch.finfo(torch.float32).min                      # empty running side: takes the block
    o0, l0 = update_out_and_lse(None, None, dev(oa), dev(la))
    assert l0.shape == (3, 40, 1) and o0.dtype == torch.float32
    o1, l1 = update_out_and_lse(o0.clone(), l0.clone(), dev(ob), dev(lb))
    rc_o, rc_l = O.lse_merge_closed_form(oa, la, ob.float(), lb)
    assert torch.allclose(o1.cpu().double(), rc_o, atol=1e-5)
    ok = rc_l > -1e30
    assert torch.allclose(l1.squeeze(-1).cpu().double()[ok], rc_l[ok], atol=1e-5)
    assert torch.equal(o1[0, :5], o0[0, :5]) and torch.equal(l1[0, :5], l0[0, :5])
    assert torch.allclose(o1[1, :5].cpu(), ob[1, :5].float(), atol=1e-6)
    # statement-for-statement restatement of the reference agrees where it is well conditioned
    ro, rl = O.update_out_and_lse(oa.clone(), la.clone().unsqueeze(-1), ob, lb)
    good = (la > -1e30) & (lb > -1e30)
    assert torch.allclose(o1.cpu()[good], ro[good], atol=1e-5)
    assert torch.allclose(l1.cpu().squeeze(-1)[good], rl.squeeze(-1)[good], atol=1e-5)


# ------------------------------------------------------------------ a11
@pytest.mark.parametrize("dtype,H,G,S,L,d,causal", [
    (torch.float32, 2, 2, 33, 33, 64, True),
    (torch.bfloat16, 2, 4, 200, 200, 128, True),
    (torch.bfloat16, 2, 4, 1, 512, 128, True),          # decode: one query sees all local keys
    (torch.float32, 1, 1, 16, 80, 32, True),            # rectangular, bottom-right aligned
    (torch.bfloat16, 1, 2, 70, 130, 128, False),
    (torch.bfloat16, 1, 2, 300, 1000, 128, True),       # several query blocks, ragged tiles
    (torch.bfloat16, 1, 1, 260, 100, 128, True),        # more queries than keys: the first 160 see nothing
    (torch.bfloat16, 1, 1, 128, 64, 128, False),        # exactly one tile
    (torch.bfloat16, 2, 2, 129, 257, 128, True),
    # the MFMA kernel's other types and head dimensions
    (torch.float16, 2, 4, 200, 200, 128, True),
    (torch.float16, 1, 2, 300, 1000, 128, True),
    (torch.float16, 2, 4, 1, 512, 128, True),
    (torch.bfloat16, 2, 2, 200, 200, 64, True),
    (torch.bfloat16, 1, 2, 300, 1000, 64, True),
    (torch.float16, 1, 2, 70, 130, 64, False),
    (torch.float16, 1, 1, 260, 100, 64, True),
    (torch.bfloat16, 1, 1, 1, 77, 64, True),
    (torch.bfloat16, 2, 2, 200, 200, 256, True),
    (torch.bfloat16, 1, 2, 300, 1000, 256, True),
    (torch.float16, 1, 2, 70, 130, 256, False),
    (torch.float16, 2, 2, 129, 257, 256, True),
    (torch.float16, 1, 3, 1, 300, 256, True),
])
def test_local_attention(ops, dtype, H, G, S, L, d, causal):
    g = gen(600)
    q = torch.randn(1, H * G, S, d, generator=g).to(dtype)
    k = torch.randn(1, H, L, d, generator=g).to(dtype)
    v = torch.randn(1, H, L, d, generator=g).to(dtype)
    out, lse = ops.local_attn_fwd(dev(q[0]), dev(k[0]), dev(v[0]), d ** -0.5, causal)
    ro, rl = O.local_attention(q, k, v, d ** -0.5, causal)
    assert_attn_close(out, lse, ro[0], rl[0], dtype, "local")
    name = ops.local_attn_fwd_kernel_name(G, S, L, d, dtype)
    mfma = dtype in (torch.bfloat16, torch.float16) and d in (64, 128, 256)
    assert name.startswith("local_attn_dense_kernel") or name == "local_attn_decode_kernel" if mfma \
        else name == "local_attn_generic_kernel", name


def test_memory_plus_local_equals_joint_softmax(ops):
    # split test on the GPU path: merge(memory bucket, local keys) == one softmax over the union
    from fast_memory_amd import Memory
    g = gen(601)
    H, G, S, N, L, d, C, Z = 2, 2, 16, 512, 16, 64, 8, 64
    keys = torch.randn(H, N, d, generator=g)
    vals = torch.randn(H, N, d, generator=g)
    A = torch.randn(H, C, d, generator=g)
    q = torch.randn(H, G * S, d, generator=g)
    kl = torch.randn(H, L, d, generator=g)
    vl = torch.randn(H, L, d, generator=g)
    mem = Memory.build(*dev(keys, vals, A), Z)
    out, lse = mem.attend_with_local(dev(q), dev(kl), dev(vl), 0.125, n_groups=G, causal=False)
    lists = mem.bucket_idx.cpu().long()
    qh = mem.hash(dev(q)).cpu().long()
    for h in range(H):
        for i in range(0, G * S, 5):
            idx = lists[h, qh[h, i]]
            kk = torch.cat([keys[h, idx], kl[h]]).double()
            vv = torch.cat([vals[h, idx], vl[h]]).double()
            s = kk @ q[h, i].double() * 0.125
            assert abs(torch.logsumexp(s, 0).item() - lse[h, i].item()) < 1e-4
            assert torch.allclose(torch.softmax(s, 0) @ vv, out[h, i].cpu().double(), atol=1e-4)


# ------------------------------------------------------------------ a12/a13
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compute_centroids(ops, dtype):
    from fast_memory_amd import compute_centroids, init_centroids
    g = gen(700)
    H, G, N, d, C, topk = 2, 2, 600, 64, 16, 8
    kq = torch.randn(H * G, N, d, generator=g).to(dtype)
    cent = O.init_centroids(C, d, dtype)
    assert torch.equal(init_centroids(C, d, "cuda", dtype).cpu(), cent)
    A = compute_centroids(dev(kq), dev(cent), C, G, topk, normalize=True).cpu()
    ref = O.compute_centroids(kq, cent, C, G, topk, normalize=True)
    assert A.shape == (C, H, d)
    assert torch.allclose(A.float().norm(dim=-1), torch.ones(C, H), atol=1e-2)
    if dtype == torch.float32:
        assert torch.allclose(A, ref, atol=1e-5), (A - ref).abs().max()
    # bf16: a near-tie of the rounded scores at the k-th place may swap one of the averaged rows against
    # the oracle's choice, so that case is held exactly elsewhere, on the GPU's own scores
    # (test_gpu_strict.py::test_compute_centroids_bf16_exact); here its shape and unit rows are checked


def test_kmeans_matches_oracle_fp32(ops):
    from fast_memory_amd import kmeans_spherical
    g = gen(701)
    H, N, d, C = 2, 3000, 64, 24
    X = O.l2_normalize(torch.randn(H, N, d, generator=g))
    init = O.l2_normalize(O.init_centroids(C, d)).unsqueeze(0).expand(H, -1, -1).contiguous()
    cent, labels = kmeans_spherical(dev(X), dev(init), 2)
    for h in range(H):
        rc, rl = O.kmeans_spherical(X[h], init[h], 2)
        agree = (labels[h].cpu().long() == rl).float().mean().item()
        assert agree > 0.999, agree                                 # fp32 vs fp64 near-ties only
        assert torch.allclose(cent[h].cpu().double(), rc, atol=1e-4)
    assert torch.allclose(cent.norm(dim=-1).cpu(), torch.ones(H, C), atol=1e-5)


def test_l2_normalize(ops):
    X = torch.randn(37, 128, generator=gen(702))
    X[3] = 0
    got = ops.l2_normalize(dev(X)).cpu()
    assert torch.allclose(got, O.l2_normalize(X), atol=1e-6)
    assert (got[3] == 0).all()


def test_l2_normalize_and_segment_mean_bf16_d128(ops):
    # the vectorised bf16 / d = 128 kernels against the oracle on the same (bf16-rounded) inputs
    from fast_memory_amd import kmeans_spherical
    g = gen(703)
    H, N, d, C = 2, 5000, 128, 37
    X = torch.randn(H, N, d, generator=g).to(torch.bfloat16)
    X[0, 7] = 0
    got = ops.l2_normalize(dev(X)).float().cpu()
    ref = O.l2_normalize(X.float())
    assert torch.allclose(got, ref, atol=4e-3, rtol=8e-3)           # one bf16 rounding of the result
    assert (got[0, 7] == 0).all()
    Xn = ref.to(torch.bfloat16)
    init = O.l2_normalize(O.init_centroids(C, d)).to(torch.bfloat16).unsqueeze(0).expand(H, -1, -1).contiguous()
    cent, labels = kmeans_spherical(dev(Xn), dev(init), 1)
    for h in range(H):
        # the centroid update on the labels the GPU assigned: mean of the members, normalised
        lab = labels[h].cpu().long()
        rc = O.kmeans_update(Xn[h].float(), lab, init[h].float())
        assert torch.allclose(cent[h].float().cpu().double(), rc.double(), atol=4e-3, rtol=8e-3)


@pytest.mark.parametrize("dtype,d,C", [(torch.bfloat16, 128, 37), (torch.float32, 64, 20), (torch.float16, 128, 11),
                                       (torch.bfloat16, 64, 9)])
def test_kmeans_on_unnormalised_rows(ops, dtype, d, C):
    """K-means on the L2-normalised keys (README.md:33-45) without a normalised copy: the assignment on the
    rows as stored (argmax_c c.x does not depend on |x|), the update dividing every member by its norm as it
    adds it -- against the oracle's update on the fp64-normalised rows for the GPU's own labels, and against the
    path that stores the normalised rows."""
    from fast_memory_amd import kmeans_spherical
    g = gen(704)
    H, N = 2, 4000
    X = (torch.randn(H, N, d, generator=g) * torch.exp(torch.randn(H, N, 1, generator=g))).to(dtype)
    X[1, 11] = 0                                            # a zero row contributes nothing
    init = O.l2_normalize(O.init_centroids(C, d)).to(dtype).unsqueeze(0).expand(H, -1, -1).contiguous()
    cent, labels = kmeans_spherical(dev(X), dev(init), 1, normalize_rows=1e-6)
    Xn = O.l2_normalize(X.double())
    tol = 1e-5 if dtype == torch.float32 else 4e-3
    for h in range(H):
        lab = labels[h].cpu().long()
        rc = O.kmeans_update(Xn[h], lab, init[h].double())
        assert torch.allclose(cent[h].float().cpu().double(), rc, atol=tol, rtol=2 * tol)
        # the labels are those of the normalised rows up to near-ties of the rounded scores
        agree = (lab == O.kmeans_assign(Xn[h], init[h].double())).float().mean().item()
        assert agree > (0.999 if dtype == torch.float32 else 0.97), agree
    cent2, labels2 = kmeans_spherical(ops.l2_normalize(dev(X)), dev(init), 1)
    assert (labels2 == labels).float().mean().item() > (0.999 if dtype == torch.float32 else 0.97)


# ------------------------------------------------------------------ golden fixture (frozen oracle outputs)
def test_library_against_the_golden_fixture(ops):
    import os
    from fast_memory_amd import (attention_hash_varlen, attention_hash_varlen_backward, update_out_and_lse)
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_fp32.npz"))
    t = {k: torch.from_numpy(gold[k]) for k in gold.files}
    H, G, d, N, C, Z, S, L = (int(x) for x in gold["dims"])
    K, V, Q, A = dev(t["K"], t["V"], t["Q"], t["A"])
    sm = d ** -0.5
    assert torch.allclose(ops.project(A, K).cpu(), t["Y"], atol=1e-5, rtol=1e-5)
    assert torch.equal(ops.argtopz(dev(t["Y"]), Z).cpu(), t["lists"])                    # bit-exact on the stored Y
    assert torch.equal(ops.qhash(A, Q).cpu(), t["qh"])
    kh, cnt, qh = dev(t["lists"].long().reshape(-1), torch.full((H, C), Z), t["qh"].long())
    out, lse = attention_hash_varlen(Q, K, V, kh, cnt, qh, sm)
    assert_attn_close(out, lse, t["out"], t["lse"], torch.float32, "fixture attention")
    lo, ll = ops.local_attn_fwd(Q.reshape(H * G, S, d), dev(t["KL"]), dev(t["VL"]), sm, True)
    assert_attn_close(lo.reshape(H, G * S, d), ll.reshape(H, G * S), t["lout"], t["llse"], torch.float32, "fixture local")
    mo, ml = update_out_and_lse(None, None, lo.reshape(H, G * S, d), ll.reshape(H, G * S))
    mo, ml = update_out_and_lse(mo, ml, out, lse)
    assert torch.allclose(mo.cpu(), t["mout"], atol=1e-4) and torch.allclose(ml.squeeze(-1).cpu(), t["mlse"], atol=1e-3)
    dq, dk, dv = attention_hash_varlen_backward(dev(t["dO"]), Q, K, V, dev(t["out"]), dev(t["lse"]), kh, cnt, qh, sm)
    for got, name in ((dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert torch.allclose(got.float().cpu(), t[name], atol=2e-4, rtol=1e-4), name


# ------------------------------------------------------------------ a15 composite, config c1
def test_config1_toy_end_to_end(ops):
    from fast_memory_amd import Memory, fit_projection
    g = gen(1001)
    d, N, C, Z, S = 64, 4096, 64, 256, 512
    K = torch.randn(1, N, d, generator=g)
    V = torch.randn(1, N, d, generator=g)
    Q = torch.randn(1, S, d, generator=g)
    A = fit_projection(dev(K), C, iters=1)
    Xn = O.l2_normalize(K[0])
    ref_A, _ = O.kmeans_spherical(Xn, O.l2_normalize(O.init_centroids(C, d)), 1)
    assert torch.allclose(A[0].cpu().double(), ref_A, atol=1e-4)
    mem = Memory.build(dev(K), dev(V), A, Z)
    Y = ops.project(A, dev(K)).cpu()
    assert torch.equal(mem.bucket_idx.cpu().long(), O.argtopz(Y, Z))            # bit-exact given the same Y
    qh, sc = ops.qhash(A, dev(Q), return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))
    out, lse = mem.attend(dev(Q), d ** -0.5)
    cnt = torch.full((1, C), Z)
    ro, rl = O.hashed_attention_gather(Q, K, V, mem.bucket_idx.cpu().long().reshape(-1), cnt, qh.cpu().long(),
                                       d ** -0.5)
    assert_attn_close(out, lse, ro, rl, torch.float32, "c1")


def test_ring_attention_masked_forward_windows(ops):
    from fast_memory_amd import ring_attention_masked_forward
    g = gen(800)
    C, H, G, S, N, Z, d, world = 6, 2, 2, 20, 256, 40, 64, 2
    q = torch.randn(1, H * G, S, d, generator=g).to(torch.bfloat16)
    kh = torch.stack([torch.stack([torch.randperm(world * N, generator=g)[:Z] for _ in range(H)]) for _ in range(C)])
    qh = torch.randint(0, C, (H, G, S), generator=g)
    for rank in range(world):
        k = torch.randn(1, H, N, d, generator=g).to(torch.bfloat16)
        v = torch.randn(1, H, N, d, generator=g).to(torch.bfloat16)
        out, lse = ring_attention_masked_forward(*dev(kh, qh, q, k, v), 0.125, rank)
        ro, rl = O.ring_attention_masked_forward(kh, qh, q, k, v, 0.125, rank)
        assert out.shape == (1, H * G, S, d) and lse.shape == (1, H * G, S)
        assert_attn_close(out[0], lse[0], ro[0], rl[0], torch.bfloat16, f"ring rank {rank}")


# ------------------------------------------------------------------ f1 backward of the gathered attention
def _assert_grad_close(got, ref, dtype, what):
    got, ref = got.float().cpu().double(), ref.double()
    if dtype == torch.float32:
        ok = torch.allclose(got, ref, atol=1e-4, rtol=1e-4)
    else:
        # bf16 inputs: products of bf16-rounded operands, gradients summed over up to hundreds of terms
        ok = torch.allclose(got, ref, atol=2e-2 * max(1.0, ref.abs().max().item()), rtol=2e-2)
    assert ok, f"{what}: max err {(got - ref).abs().max().item():.3e} (ref max {ref.abs().max().item():.3e})"


@pytest.mark.parametrize("dtype,B,S,N,C,Z,d", [
    (torch.float32, 2, 70, 300, 6, 40, 64),
    (torch.float32, 1, 24, 1024, 8, 16, 16),             # the reference's small test shape (tk:500)
    (torch.bfloat16, 2, 200, 2000, 12, 150, 128),
    (torch.bfloat16, 1, 130, 700, 3, 333, 128),          # more than 64 queries per bucket: several items
    (torch.float16, 2, 200, 2000, 12, 150, 128),         # fp16 on the MFMA kernel
    (torch.float16, 1, 130, 700, 3, 333, 128),
    (torch.float16, 2, 70, 300, 6, 40, 64),              # fp16 on the generic kernel
])
def test_hash_attention_backward(ops, dtype, B, S, N, C, Z, d):
    from fast_memory_amd import attention_hash_varlen, attention_hash_varlen_backward
    q, k, v, kh, cnt, qh = make_attn_case(1200 + S, B, S, N, C, Z, d, dtype, window="ref", std=0.7)
    dout = (torch.randn(B, S, d, generator=gen(1300 + S)) * 0.5).to(dtype)
    sm = d ** -0.5
    args = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(*args, sm)
    dq, dk, dv = attention_hash_varlen_backward(dev(dout), args[0], args[1], args[2], out, lse, args[3], args[4],
                                                args[5], sm)
    assert dq.dtype == dtype and dk.dtype == torch.float32 and dk.shape == k.shape
    # oracle on the same (rounded) inputs and on the GPU's own out / lse
    rq, rk, rv = O.hashed_attention_backward_gather(q.float(), k.float(), v.float(), kh, cnt, qh, out.float().cpu(),
                                                    lse.cpu(), dout.float(), sm)
    _assert_grad_close(dq, rq, dtype, "dq")
    _assert_grad_close(dk, rk, dtype, "dk")
    _assert_grad_close(dv, rv, dtype, "dv")
    empty = lse.cpu() < -1e30
    assert (dq.float().cpu()[empty] == 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_mfma_and_generic_agree(ops, dtype):
    from fast_memory_amd import attention_hash_varlen, attention_hash_varlen_backward
    q, k, v, kh, cnt, qh = make_attn_case(1500, 2, 300, 3000, 9, 500, 128, dtype, window="ref", std=0.7)
    qh[0, :150] = 2                                             # a bucket with several 16-query tiles and items
    dout = (torch.randn(2, 300, 128, generator=gen(1501)) * 0.5).to(dtype)
    args = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(*args, 128 ** -0.5)
    call = lambda: attention_hash_varlen_backward(dev(dout), args[0], args[1], args[2], out, lse, args[3], args[4],
                                                  args[5], 128 ** -0.5)
    dq1, dk1, dv1 = call()
    ops.force_generic_kernels(True)
    try:
        dq2, dk2, dv2 = call()
    finally:
        ops.force_generic_kernels(False)
    for a, b, name in ((dq1, dq2, "dq"), (dk1, dk2, "dk"), (dv1, dv2, "dv")):
        a, b = a.float(), b.float()
        assert torch.allclose(a, b, atol=2e-2 * max(1.0, b.abs().max().item()), rtol=2e-2), \
            f"{name}: {(a - b).abs().max().item():.3e} vs max {b.abs().max().item():.3e}"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ws_bytes,C", [(24 << 30, 10), (1 << 20, 10),    # everything in one pass; one row per pass
                                        (24 << 30, 16)])                   # fewer queries per bucket: the two-tile kernel
def test_backward_staged_equals_atomic_and_oracle(ops, ws_bytes, C, dtype):
    """The backward without atomics (per-bucket partial rows, then a sum per key over the inverted lists)
    against the atomic path and the oracle: buckets with several query tiles (passes of one, two and four
    tiles; the launch takes the four-tile kernel above 24 queries per bucket on average), buckets nobody
    hashed to, ragged and empty lists, keys listed by no bucket."""
    from fast_memory_amd import attention_hash_varlen
    B, S, N, Z, d = 3, 260, 1500, 200, 128
    q, k, v, kh, cnt, qh = make_attn_case(1600, B, S, N, C, Z, d, dtype, window="ref", std=0.7)
    qh[0, :120] = 2                                             # 120 queries in one bucket: 8 tiles
    qh[qh == 7] = 8                                             # bucket 7 receives no query
    qh[1] = 4                                                   # one row hashes everything to one bucket
    dout = (torch.randn(B, S, d, generator=gen(1601)) * 0.5).to(dtype)
    sm = d ** -0.5
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(qd, kd, vd, khd, cntd, qhd, sm)
    lists, counts = khd.int().contiguous(), cntd.int().contiguous()
    off = ops.bucket_offsets(counts)
    groups = ops.group_queries(qhd.int().contiguous(), C)
    inv = ops.inverse_index(lists, off, counts, N)
    # the inverse index is exactly the inversion of the lists
    ko, ip = inv.key_off.cpu().long(), inv.inv_pos.cpu().long()
    flat = kh.long()
    row_of_pos = torch.repeat_interleave(torch.arange(B * C), cnt.reshape(-1)) // C
    keys_sorted = row_of_pos[ip] * N + flat[ip]
    assert torch.equal(keys_sorted, torch.sort(row_of_pos * N + flat, stable=True).values)
    assert torch.equal(ip, torch.sort(row_of_pos * N + flat, stable=True).indices)
    assert torch.equal(ko, torch.searchsorted(keys_sorted, torch.arange(B * N + 1)))
    dq1, dk1, dv1 = ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm,
                                             workspace_bytes=ws_bytes)
    dq2, dk2, dv2 = ops.hash_attn_bwd(qd, kd, vd, lists, off, counts, groups, out, lse, dev(dout), sm)
    rq, rk, rv = O.hashed_attention_backward_gather(q.float(), k.float(), v.float(), kh, cnt, qh, out.float().cpu(),
                                                    lse.cpu(), dout.float(), sm)
    for got, other, ref, name in ((dq1, dq2, rq, "dq"), (dk1, dk2, rk, "dk"), (dv1, dv2, rv, "dv")):
        _assert_grad_close(got, ref, dtype, name + " (staged vs oracle)")
        _assert_grad_close(got, other.float().cpu(), dtype, name + " (staged vs atomic)")
    # a fixed summation order: bit-identical from run to run, and when the rows go through one at a time
    dq3, dk3, dv3 = ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm,
                                             workspace_bytes=24 << 30)
    assert torch.equal(dk1, dk3) and torch.equal(dv1, dv3) and torch.equal(dq1, dq3)
    # accumulation into given buffers
    dk0 = torch.ones_like(dk1)
    _, dk4, _ = ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm, dk=dk0)
    assert dk4 is dk0 and torch.allclose(dk4, dk1 + 1.0, atol=1e-6)


def test_memory_attend_backward_against_autograd(ops):
    """Memory.attend_backward (staged form, inverse index kept by the memory) against torch autograd of a dense
    softmax over each query's bucket, and the kept index is rebuilt after an append."""
    from fast_memory_amd import Memory
    g = gen(1650)
    H, N, C, Z, S, d = 2, 600, 5, 128, 40, 128
    K = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    V = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
    q = (torch.randn(H, S, d, generator=g) * 0.5).to(torch.bfloat16)
    dout = (torch.randn(H, S, d, generator=g) * 0.5).to(torch.bfloat16)
    mem = Memory.build(*dev(K, V, A), Z, keep_values=True)
    qd = dev(q)
    qh = mem.hash(qd)
    out, lse = mem.attend(qd, d ** -0.5, q_hash=qh)
    dq, dk, dv = mem.attend_backward(dev(dout), qd, out, lse, d ** -0.5, q_hash=qh)
    inv0 = mem.inverse_index()
    assert mem.inverse_index() is inv0                                   # kept
    # autograd reference in fp64 on the same lists
    lists, qhc = mem.bucket_idx.cpu().long(), qh.cpu().long()
    Kr, Vr, qr = K.double().requires_grad_(), V.double().requires_grad_(), q.double().requires_grad_()
    outs = []
    for h in range(H):
        idx = lists[h][qhc[h]]                                            # [S, Z]
        s = torch.einsum("sd,szd->sz", qr[h], Kr[h][idx]) * d ** -0.5
        outs.append(torch.einsum("sz,szd->sd", torch.softmax(s, -1), Vr[h][idx]))
    torch.stack(outs).backward(dout.double())
    _assert_grad_close(dq, qr.grad, torch.bfloat16, "dq")
    _assert_grad_close(dk, Kr.grad, torch.bfloat16, "dk")
    _assert_grad_close(dv, Vr.grad, torch.bfloat16, "dv")
    mem.append(dev(K[:, :50].contiguous()), dev(V[:, :50].contiguous()))
    inv1 = mem.inverse_index()
    assert inv1 is not inv0 and inv1.key_off.numel() == H * (N + 50) + 1  # rebuilt for the longer memory


def test_backward_staged_blocks_through_lds_same_bits(ops):
    """The first pass of the staged backward over a bucket (up to 32 queries) takes its key blocks through LDS,
    requested a block ahead; the same pass with the blocks loaded into registers (the diagnostic switch) gives
    the same bits.  Lists of many blocks, ragged and empty ones, lengths that are no multiple of a block or
    of a pair of blocks; buckets of 1 to 40 queries (below 17 and above 32 other passes run); twice in a row."""
    B, S, N, C, Z, d = 2, 900, 9000, 40, 1999, 128
    q, k, v, kh, cnt, qh = make_attn_case(1610, B, S, N, C, Z, d, torch.bfloat16, window="ref", std=0.7)
    cnt[0, 3], cnt[0, 4], cnt[1, 5], cnt[1, 6] = 0, 1, 33, 64
    dout = (torch.randn(B, S, d, generator=gen(1611)) * 0.5).to(torch.bfloat16)
    sm = d ** -0.5
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    from fast_memory_amd import attention_hash_varlen
    out, lse = attention_hash_varlen(qd, kd, vd, khd, cntd, qhd, sm)
    lists, counts = khd.int().contiguous(), cntd.int().contiguous()
    off = ops.bucket_offsets(counts)
    groups = ops.group_queries(qhd.int().contiguous(), C)
    per_bucket = groups.bin_count.reshape(-1)
    assert S > 12 * C                                           # the launch takes the form with the LDS blocks
    assert int(((per_bucket > 16) & (per_bucket <= 32)).sum()) >= 10 and int((per_bucket > 32).sum()) >= 1
    inv = ops.inverse_index(lists, off, counts, N)
    run = lambda: ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm)
    a, b = run(), run()
    ops.grouped_forward_kernel("bwd-register-blocks")
    try:
        c = run()
    finally:
        ops.grouped_forward_kernel(None)
    for x, y, z, name in zip(a, b, c, ("dq", "dk", "dv")):
        assert torch.equal(x, y), name + ": two runs differ"
        assert torch.equal(x, z), name + ": blocks through LDS and blocks in registers differ"
    rq, rk, rv = O.hashed_attention_backward_gather(q.float(), k.float(), v.float(), kh, cnt, qh, out.float().cpu(),
                                                    lse.cpu(), dout.float(), sm)
    for got, ref, name in ((a[0], rq, "dq"), (a[1], rk, "dk"), (a[2], rv, "dv")):
        _assert_grad_close(got, ref, torch.bfloat16, name)


def _inverse_by_stable_sort(flat_lists, rows, H, N):
    flat = flat_lists.long() + rows * N
    order = torch.sort(flat, stable=True).indices
    key_off = torch.zeros(H * N + 1, dtype=torch.int64, device=flat.device)
    key_off[1:] = torch.cumsum(torch.bincount(flat, minlength=H * N), 0)
    return key_off.int(), order.int()


@pytest.mark.parametrize("H,N,C,Z", [(2, 5000, 24, 333), (3, 700, 5, 40), (1, 256, 3, 256), (2, 70000, 130, 900),
                                     (4, 131072, 64, 4096), (1, 3000, 70000, 3)])
def test_inverse_index_by_transposition_and_by_sort(ops, H, N, C, Z):
    """Lists in ascending key order are inverted by a transposition over key ranges, any others by a stable
    radix sort; both equal a stable sort of (row, key) over the flat positions.  Ragged lists with empty
    ones, runs of a key range longer than a group of lanes (Z = N), keys that no list names, N off the range
    size; then the same lists out of order, and with one repeated key, which take the sort."""
    g = torch.Generator(device="cuda").manual_seed(1700 + H)
    # strictly ascending keys: a prefix sum of gaps >= 1 that stays below N
    hi = max(1, 2 * (N // Z) - 1) if N > Z else 1
    gaps = torch.randint(1, hi + 1, (H, C, Z), device="cuda", generator=g, dtype=torch.int32)
    gaps[..., 0] = torch.randint(1, max(2, N // (4 * Z)) + 1, (H, C), device="cuda", generator=g, dtype=torch.int32)
    lists = torch.cumsum(gaps, -1, dtype=torch.int32) - 1
    lists = torch.minimum(lists, (N - Z + torch.arange(Z, device="cuda", dtype=torch.int32)).expand(H, C, Z))
    assert int(lists.max()) < N and bool((lists[..., 1:] > lists[..., :-1]).all())
    cnt = torch.randint(0, Z + 1, (H, C), device="cuda", generator=g, dtype=torch.int32)
    cnt[0, 0] = 0
    cnt[-1, -1] = Z
    cnt[0, -1] = Z
    off = ops.bucket_offsets(cnt)
    mask = torch.arange(Z, device="cuda")[None, None, :] < cnt[..., None]
    rows = torch.arange(H, device="cuda")[:, None, None].expand(H, C, Z)[mask]
    flat_lists = lists[mask].contiguous()
    inv = ops.inverse_index(flat_lists, off, cnt, N)
    assert ops.last_inverse_info["path"] == ("transposition" if C <= 65535 else "sort")   # 16-bit counters per key
    ko, ip = _inverse_by_stable_sort(flat_lists, rows, H, N)
    assert torch.equal(inv.key_off, ko) and torch.equal(inv.inv_pos, ip)
    assert inv.row_pos == tuple(off[:, 0].tolist()) + (flat_lists.numel(),)
    # the same entries in another order inside every list
    shuffled = torch.where(mask, lists, torch.full_like(lists, N))               # unlisted entries sort last
    perm = torch.rand(H, C, Z, device="cuda", generator=g).masked_fill(~mask, 2.0).argsort(-1)
    flat_shuffled = torch.gather(shuffled, -1, perm)[mask].contiguous()
    inv = ops.inverse_index(flat_shuffled, off, cnt, N)
    assert ops.last_inverse_info["path"] == "sort"
    ko, ip = _inverse_by_stable_sort(flat_shuffled, rows, H, N)
    assert torch.equal(inv.key_off, ko) and torch.equal(inv.inv_pos, ip)
    # one key twice in one list: not the order the transposition takes
    twice = flat_lists.clone()
    last = int(off[-1, -1])
    twice[last + 1] = twice[last]
    inv = ops.inverse_index(twice, off, cnt, N)
    assert ops.last_inverse_info["path"] == "sort"
    ko, ip = _inverse_by_stable_sort(twice, rows, H, N)
    assert torch.equal(inv.key_off, ko) and torch.equal(inv.inv_pos, ip)


def test_ring_attention_masked_backward_with_merged_result(ops):
    # memory part of a merged attention: out / lse passed to the backward are those of the softmax over
    # bucket keys and local keys together; checked against autograd through a dense fp64 evaluation
    from fast_memory_amd import ring_attention_masked_backward, ring_attention_masked_forward, update_out_and_lse
    g = gen(1400)
    C, H, G, S, N, Z, d, L = 5, 2, 2, 12, 200, 30, 64, 9
    sm = 0.125
    q = torch.randn(1, H * G, S, d, generator=g)
    k = torch.randn(1, H, N, d, generator=g)
    v = torch.randn(1, H, N, d, generator=g)
    kl = torch.randn(1, H, L, d, generator=g)
    vl = torch.randn(1, H, L, d, generator=g)
    w = torch.randn(1, H * G, S, d, generator=g)
    kh = torch.stack([torch.stack([torch.randperm(N, generator=g)[:Z] for _ in range(H)]) for _ in range(C)])
    qh = torch.randint(0, C, (H, G, S), generator=g)
    # dense fp64 forward of the union softmax with autograd
    qd, kd, vd = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    vis = torch.zeros(H, G, S, N, dtype=torch.bool)
    for h in range(H):
        for gg in range(G):
            for i in range(S):
                vis[h, gg, i, kh[qh[h, gg, i], h]] = True
    s_m = (torch.einsum('hgid,hjd->hgij', qd[0].view(H, G, S, d), kd[0]) * sm).masked_fill(~vis, -float("inf"))
    s_l = torch.einsum('hgid,hjd->hgij', qd[0].view(H, G, S, d), kl[0].double()) * sm
    P = torch.softmax(torch.cat([s_m, s_l], -1), -1)
    o = torch.einsum('hgij,hjd->hgid', P[..., :N], vd[0]) + torch.einsum('hgij,hjd->hgid', P[..., N:], vl[0].double())
    (o.reshape(1, H * G, S, d) * w.double()).sum().backward()
    # GPU: forward of both parts, merge, backward of the memory part with the merged result
    mo, ml = ring_attention_masked_forward(*dev(kh, qh, q, k, v), sm, 0)
    lo, ll = ops.local_attn_fwd(dev(q[0]), dev(kl[0]), dev(vl[0]), sm, False)
    out, lse = update_out_and_lse(None, None, lo.unsqueeze(0), ll.unsqueeze(0))
    out, lse = update_out_and_lse(out.contiguous(), lse.contiguous(), mo, ml)
    assert torch.allclose(out.cpu().double(), o.detach().reshape(1, H * G, S, d), atol=1e-4)
    dq, dk, dv = ring_attention_masked_backward(*dev(kh, qh), torch.arange(H), dev(w), dev(q), dev(k), dev(v),
                                                out.to(q.dtype), lse.squeeze(-1), sm, 0)
    assert torch.allclose(dk.cpu().double(), kd.grad, atol=2e-4, rtol=1e-4)
    assert torch.allclose(dv.cpu().double(), vd.grad, atol=2e-4, rtol=1e-4)
    rq, _, _ = O.ring_attention_masked_backward_ref(kh, qh, w, q, k, v, o.detach().reshape(q.shape),
                                                    torch.logsumexp(torch.cat([s_m, s_l], -1), -1).detach().reshape(1, H * G, S),
                                                    sm, 0)
    assert torch.allclose(dq.cpu().double(), rq, atol=2e-4, rtol=1e-4)


# ------------------------------------------------------------------ f2 target of the learned projection
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_calc_ref_centroids(ops, dtype):
    from fast_memory_amd import calc_ref_centroids, learn_emb_proj
    g = gen(1600)
    B, H, G, S, N, d = 1, 2, 2, 50, 700, 128 if dtype == torch.bfloat16 else 32
    q = torch.randn(B, H * G, S, d, generator=g).to(dtype)
    k = torch.randn(B, H, N, d, generator=g).to(dtype)
    got = calc_ref_centroids(dev(q), dev(k), workspace_bytes=1 << 20)      # small table: several row chunks
    assert got.shape == (B, H, G, N, d) and got.dtype == dtype
    ref = O.calc_ref_centroids(q.float(), k.float())
    diff = (got.float().cpu().double() - ref).abs().amax(-1)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    # a key whose score sits at a query's rank-128 boundary can flip on fp32-vs-fp64 rounding of that score
    assert (diff <= tol).double().mean().item() > 0.995, (diff > tol).sum().item()
    kq = torch.randn(B, N, H * G * d, generator=g).to(dtype)
    kqn, loss = learn_emb_proj(dev(kq), dev(q), dev(k))
    assert kqn.shape == (B, H * G, N, d)
    kq_ref = kq.float().view(B, N, H * G, d).permute(0, 2, 1, 3).reshape(B, H, G, N, d)
    kq_ref = kq_ref / kq_ref.norm(dim=-1, keepdim=True).clamp(min=1e-6)
    ref_loss = torch.nn.functional.mse_loss(kq_ref.double(), ref).item()
    assert abs(loss.item() - ref_loss) < (1e-5 if dtype == torch.float32 else 2e-3) * max(1.0, ref_loss)


# ------------------------------------------------------------------ f3 persistent memory, incremental append
@pytest.mark.parametrize("dtype,H,C,N0,M,Z,d", [
    (torch.float32, 2, 9, 500, 77, 64, 32),
    (torch.bfloat16, 2, 20, 3000, 1000, 256, 128),
    (torch.bfloat16, 1, 6, 40, 30, 64, 128),              # the lists are not full yet: they grow, then fill
    (torch.bfloat16, 1, 4, 2000, 9000, 8192, 128),        # more new keys than old ones, long lists
    (torch.bfloat16, 2, 20, 3000, 1, 256, 128),           # few keys into full lists: only the rows they enter are touched
    (torch.bfloat16, 2, 20, 3000, 40, 256, 128),
    (torch.float32, 1, 9, 500, 3, 64, 32),
])
def test_append_equals_rebuild(ops, dtype, H, C, N0, M, Z, d, tmp_path):
    from fast_memory_amd import Memory
    g = gen(1700 + M)
    K = torch.randn(H, N0 + 2 * M, d, generator=g).to(dtype)
    K[:, N0 + min(3, M - 1)] = K[:, 5]                       # a new key that ties with an old one: the old one wins
    V = torch.randn(H, N0 + 2 * M, d, generator=g).to(dtype)
    A = torch.randn(H, C, d, generator=g).to(dtype)
    Kd, Vd, Ad = dev(K, V, A)
    mem = Memory.build(Kd[:, :N0], Vd[:, :N0], Ad, Z, keep_values=True)
    Y0 = ops.project(Ad, Kd[:, :N0].contiguous())
    assert torch.equal(mem.bucket_val, torch.gather(Y0, 2, mem.bucket_idx.long()) + 0.0)   # the values are Y's
    for step in range(2):                                    # two appends in a row
        n1 = N0 + (step + 1) * M
        before = mem.bucket_idx
        mem.append(Kd[:, n1 - M:n1], Vd[:, n1 - M:n1])
        assert (mem.bucket_idx is before) == (n1 - M >= Z)      # full lists are updated in place
        ref = Memory.build(Kd[:, :n1], Vd[:, :n1], Ad, Z, keep_values=True)
        assert torch.equal(mem.bucket_idx, ref.bucket_idx), f"append {step}: lists differ from a rebuild"
        assert torch.equal(mem.bucket_val, ref.bucket_val)
        assert torch.equal(mem.keys, Kd[:, :n1]) and torch.equal(mem.bucket_cnt, ref.bucket_cnt)
    # and the oracle on the final state
    Y = ops.project(Ad, Kd).cpu()
    assert torch.equal(mem.bucket_idx.cpu().long(), O.argtopz(Y, Z))
    # persistence: a saved and reloaded memory answers queries bit-identically
    path = str(tmp_path / "mem.safetensors")
    mem.save(path)
    mem2 = Memory.load(path, "cuda")
    assert mem2.Z == Z and torch.equal(mem2.bucket_idx, mem.bucket_idx) and torch.equal(mem2.bucket_val, mem.bucket_val)
    q = dev(torch.randn(H, 33, d, generator=g).to(dtype))
    o1, l1 = mem.attend(q, d ** -0.5)
    o2, l2 = mem2.attend(q, d ** -0.5)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)


def test_append_falls_back_to_rebuild_when_a_bucket_takes_too_many(ops):
    from fast_memory_amd import Memory
    g = gen(1750)
    H, C, N0, M, Z, d = 1, 3, 20000, 12000, 16384, 128
    K = (torch.randn(H, N0 + M, d, generator=g) * 0.1)
    A = torch.randn(H, C, d, generator=g)
    K[0, N0:] += A[0, 1] / A[0, 1].norm() * 3.0            # every new key lands at the top of bucket 1
    K, A = K.to(torch.bfloat16), A.to(torch.bfloat16)
    V = torch.zeros_like(K)
    Kd, Vd, Ad = dev(K, V, A)
    mem = Memory.build(Kd[:, :N0], Vd[:, :N0], Ad, Z, keep_values=True)
    assert ops.index_append(Ad, Kd[:, N0:].contiguous(), N0, mem.bucket_idx, mem.bucket_val, Z) is None
    snap = mem.bucket_idx.clone()
    mem_b = Memory.build(Kd[:, :N0 - 1], Vd[:, :N0 - 1], Ad, Z, keep_values=True)
    mem_b.append(Kd[:, N0 - 1:N0], Vd[:, N0 - 1:N0])                 # one key, in place: almost every bucket untouched
    assert torch.equal(mem_b.bucket_idx, snap) and torch.equal(mem_b.bucket_val, mem.bucket_val)
    mem.append(Kd[:, N0:], Vd[:, N0:])
    ref = ops.build_index(Ad, Kd, Z)
    assert torch.equal(mem.bucket_idx, ref)


# ------------------------------------------------------------------ a1+a2 fused build
def _clustered_keys(g, H, N, d, n_clusters=64, spread=0.5):
    cen = torch.randn(H, n_clusters, d, generator=g)
    comp = torch.randint(0, n_clusters, (H, N), generator=g)
    x = torch.gather(cen, 1, comp[..., None].expand(-1, -1, d)) + spread * torch.randn(H, N, d, generator=g)
    return x.to(torch.bfloat16)


def test_fused_build_bit_identical_to_unfused(ops):
    g = gen(900)
    H, C, N, d, Z = 2, 70, 70001, 128, 512                # ragged C (one partial wave) and a key tail
    K = _clustered_keys(g, H, N, d)
    A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    assert _libmod().load().fm_build_index_fused_workspace(H, C, N, d, Z, 1) > 0
    fused = ops.build_index(Ad, Kd, Z, fused=True)
    assert ops.last_build_info["path"] == "fused" and ops.last_build_info["rows_unresolved"] == 0
    unfused = ops.build_index(Ad, Kd, Z, fused=False)
    assert torch.equal(fused, unfused)
    Y = ops.project(Ad, Kd).cpu()
    assert torch.equal(fused.cpu().long(), O.argtopz(Y, Z))


@pytest.mark.parametrize("H,C,N,Z", [(1, 513, 65536 + 31, 64),        # one bucket past a 512-bucket slab, ragged key tile
                                     (3, 1024, 98304, 4096),           # three splits' worth of whole tiles
                                     (2, 600, 131072 + 1, 2000),       # Z not a power of two, one key past a tile
                                     (1, 64, 65536, 8192),             # the longest list N/8 allows here
                                     (8, 256, 32768, 1024),            # the prefill chunk's extents
                                     (2, 130, 16384, 2048),            # the shortest memory the fused build takes, Z = N/8
                                     (3, 1024, 20001, 64)])            # ... a ragged one, the shortest lists
def test_fused_build_shapes(ops, H, C, N, Z):
    g = gen(910 + C)
    K = _clustered_keys(g, H, N, 128)
    A = torch.randn(H, C, 128, generator=g).to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    fused, fv = ops.build_index(Ad, Kd, Z, fused=True, return_values=True)
    assert ops.last_build_info["path"] == "fused" and ops.last_build_info["rows_unresolved"] == 0
    unfused, uv = ops.build_index(Ad, Kd, Z, fused=False, return_values=True)
    assert torch.equal(fused, unfused) and torch.equal(fv.view(torch.int32), uv.view(torch.int32))


def test_fused_build_many_rows_with_short_lists(ops):
    """32 768 rows whose thresholds come from few sample values (rank 61 of a 4096-key sample): a threshold
    that spreads by a relative 1 / sqrt(rank) must neither overflow the candidate segments nor leave more rows
    to repair than can be repaired -- the build stays on the fused path and gives the unfused lists."""
    H, C, N, Z = 8, 4096, 262144, 2048
    g = torch.Generator(device="cuda").manual_seed(915)
    K = (torch.randn(H, N, 128, generator=g, device="cuda") * 0.6).to(torch.bfloat16)
    A = torch.nn.functional.normalize(torch.randn(H, C, 128, generator=g, device="cuda"), dim=-1).to(torch.bfloat16)
    fused = ops.build_index(A, K, Z, fused=True)
    info = dict(ops.last_build_info)
    assert info["path"] == "fused" and info["rows_unresolved"] == 0 and info["rows_repaired"] <= 24, info
    assert torch.equal(fused, ops.build_index(A, K, Z, fused=False))


@pytest.mark.parametrize("dtype,H,C,N,Z,runs", [
    (torch.bfloat16, 2, 1024, 65536 + 77, 1100, False),   # pass rate ~2 %: four rounds, one pass; a ragged key tile
    (torch.bfloat16, 1, 900, 131072, 6000, False),        # ~6 %: seven rounds, three passes; a partial last wave
    (torch.float16, 2, 2048, 98304, 3000, False),         # ~4 %: six rounds, two passes; two slabs
    (torch.bfloat16, 1, 1024, 70000, 1100, True),         # the keys of a cluster side by side: a bucket takes whole
    (torch.float16, 2, 1024, 131072, 2500, True),         # groups of 16 keys, more than the rounds and passes hold
])
def test_fused_build_filter_forms_agree(ops, dtype, H, C, N, Z, runs):
    """The filter that issues its epilogue between its MFMAs (fused_filter_ping_kernel; slabs of 1024 buckets,
    a queue of candidates per wave, fixed numbers of rounds and passes picked from the expected pass rate, loops
    for what they do not reach) against the filter it replaces there and against the unfused build: the same
    lists and values.  With the keys of a cluster in consecutive positions the buckets near it take most keys of
    a group at once, which overflows the rounds and the passes."""
    lib = _libmod().load()
    g = gen(930 + C + Z)
    if runs:
        cen = torch.randn(H, 48, 128, generator=g)
        comp = torch.sort(torch.randint(0, 48, (H, N), generator=g), dim=1).values
        K = (torch.gather(cen, 1, comp[..., None].expand(-1, -1, 128)) + 0.3 * torch.randn(H, N, 128, generator=g)).to(dtype)
        A = (cen[:, torch.arange(C) % 48] + 0.7 * torch.randn(H, C, 128, generator=g)).to(dtype)
    else:
        K = _clustered_keys(g, H, N, 128).to(dtype)
        A = torch.randn(H, C, 128, generator=g).to(dtype)
    Ad, Kd = dev(A, K)
    dt = {torch.bfloat16: 1, torch.float16: 2}[dtype]
    assert lib.fm_build_index_fused_kernel(H, C, N, 128, Z, dt) == b"fused_filter_ping_kernel"
    new, nv = ops.build_index(Ad, Kd, Z, fused=True, return_values=True)
    info = dict(ops.last_build_info)
    assert info["path"] == "fused" and info["rows_unresolved"] == 0, info
    lib.fm_debug_fused_filter(1)
    try:
        assert lib.fm_build_index_fused_kernel(H, C, N, 128, Z, dt) == b"fused_filter_wide_kernel"
        old, ov = ops.build_index(Ad, Kd, Z, fused=True, return_values=True)
        assert ops.last_build_info["path"] == "fused"
    finally:
        lib.fm_debug_fused_filter(0)
    assert torch.equal(new, old) and torch.equal(nv.view(torch.int32), ov.view(torch.int32))
    unfused, uv = ops.build_index(Ad, Kd, Z, fused=False, return_values=True)
    assert torch.equal(new, unfused) and torch.equal(nv.view(torch.int32), uv.view(torch.int32))


def test_fused_build_repairs_rows_whose_sampled_threshold_missed(ops):
    g = gen(901)
    H, C, N, d, Z = 1, 40, 131072, 128, 1024               # sample stride 4: keys 0,4,8,... are sampled
    K = (0.3 * torch.randn(H, N, d, generator=g))
    A = torch.randn(H, C, d, generator=g)
    A = A / A.norm(dim=-1, keepdim=True)
    samp = torch.arange(0, N, 4)
    off = torch.arange(1, N, 4)
    K[0, off[:20000]] += 3.0 * A[0, 3]                      # row 3: many large values the sample never sees
    K[0, samp[:600]] += 3.0 * A[0, 7]                       # row 7: the sample over-represents the large values
    K, A = K.to(torch.bfloat16), A.to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    fused = ops.build_index(Ad, Kd, Z, fused=True)
    info = dict(ops.last_build_info)
    assert info["path"] == "fused" and info["rows_unresolved"] == 0 and info["rows_repaired"] >= 2, info
    assert torch.equal(fused, ops.build_index(Ad, Kd, Z, fused=False))


def test_fused_build_falls_back_when_too_many_rows_miss(ops):
    g = gen(902)
    H, C, N, d, Z = 1, 100, 65536, 128, 256                # stride 2: even keys sampled
    A = torch.randn(H, C, d, generator=g)
    K = 0.1 * torch.randn(H, N, d, generator=g)
    K[0, 1::2] += 2.0 * A[0].sum(0) / 10                    # every row's large values sit on unsampled keys
    K, A = K.to(torch.bfloat16), A.to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    lists = ops.build_index(Ad, Kd, Z)
    assert torch.equal(lists, ops.build_index(Ad, Kd, Z, fused=False))
    Y = ops.project(Ad, Kd).cpu()
    assert torch.equal(lists.cpu().long(), O.argtopz(Y, Z))


def _libmod():
    from fast_memory_amd import _lib
    return _lib


# ------------------------------------------------------------------ MFMA kernels vs generic kernels
def test_mfma_and_generic_attention_agree(ops):
    q, k, v, kh, cnt, qh = make_attn_case(30, 3, 500, 8192, 40, 700, 128, torch.bfloat16, window="all", std=1.0)
    qh[1, :200] = 7
    args = dev(q, k, v, kh.int(), cnt.int(), qh.int())
    o1, l1 = ops.attention_hash_varlen_i32(*args, 128 ** -0.5)
    ops.force_generic_kernels(True)
    try:
        o2, l2 = ops.attention_hash_varlen_i32(*args, 128 ** -0.5)
    finally:
        ops.force_generic_kernels(False)
    assert torch.allclose(o1.float(), o2.float(), atol=2e-2, rtol=1e-2)
    assert (l1 - l2).abs().max().item() < 1e-3


# ------------------------------------------------------------------ reduced copies of the benchmark workloads
@pytest.mark.parametrize("name,N,S,H,C,Z", [
    ("c2", 4096, 64, 2, 32, 256),            # unfused build (N < 65536)
    ("c5", 65536, 16, 1, 64, 1024),          # fused build, local keys + merge
])
def test_reduced_benchmark_workloads_end_to_end(ops, name, N, S, H, C, Z):
    from fast_memory_amd import Memory, fit_projection, synth
    cfg = synth.CONFIGS[name]
    wl = synth.make_workload(cfg, "cpu", N=N, S=S, H=H)
    keys, vals, q = dev(wl.keys, wl.values, wl.queries)
    A = fit_projection(keys, C, iters=cfg.kmeans_iters)
    mem = Memory.build(keys, vals, A, Z)
    Y = ops.project(A, keys).cpu()
    assert torch.equal(mem.bucket_idx.cpu().long(), O.argtopz(Y, Z))
    qh, sc = ops.qhash(A, q, return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))
    scale = cfg.d ** -0.5
    out, lse = mem.attend(q, scale, q_hash=qh)
    cnt = torch.full((H, C), Z)
    ro, rl = O.hashed_attention_gather(wl.queries, wl.keys, wl.values, mem.bucket_idx.cpu().long().reshape(-1),
                                       cnt, qh.cpu().long(), scale)
    assert_attn_close(out, lse, ro, rl, cfg.dtype, name)
    if wl.k_local is not None:
        G = cfg.G
        L = wl.k_local.shape[1]
        kl, vl = wl.k_local[:, L - S:], wl.v_local[:, L - S:]          # S local keys, causal against S tokens
        mo, ml = mem.attend_with_local(q, dev(kl.contiguous()), dev(vl.contiguous()), scale, n_groups=G, causal=True)
        lo, ll = O.local_attention(wl.queries.reshape(1, H * G, S, cfg.d), kl.reshape(1, H, S, cfg.d),
                                   vl.reshape(1, H, S, cfg.d), scale, True)
        eo, el = O.lse_merge_closed_form(lo[0].reshape(H, G * S, cfg.d).float(), ll[0].reshape(H, G * S),
                                         ro.float(), rl)
        assert torch.allclose(mo.cpu().double(), eo, atol=2e-2, rtol=1e-2)
        assert (ml.cpu().double() - el).abs().max().item() < 2e-3


# ------------------------------------------------------------------ varlen decode batch (config 3 shape)
def test_decode_batch_of_different_memories(ops):
    from fast_memory_amd import Memory, MemoryBatch
    g = gen(950)
    H, G, d = 2, 4, 128
    shapes = [(3000, 55, 219), (5000, 71, 283), (4096, 64, 256), (700, 26, 106)]       # (N, C~sqrt N, Z~4 sqrt N)
    mems, cpu = [], []
    for N, C, Z in shapes:
        K = torch.randn(H, N, d, generator=g).to(torch.bfloat16)
        V = torch.randn(H, N, d, generator=g).to(torch.bfloat16)
        A = torch.randn(H, C, d, generator=g)
        A = (A / A.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
        mems.append(Memory.build(*dev(K, V, A), Z))
        cpu.append((K, V, A))
    batch = MemoryBatch(mems)
    q = (torch.randn(len(shapes), H, G, d, generator=g) * 2).to(torch.bfloat16)
    q[1, 0, 2] = q[1, 0, 0]                                          # two queries of a row share a bucket
    out, lse, h, scores = batch.attend(dev(q), 128 ** -0.5, return_scores=True)
    out, lse, h, scores = out.cpu(), lse.cpu(), h.cpu().long(), scores.cpu()
    a_off = 0
    for s, ((N, C, Z), (K, V, A), mem) in enumerate(zip(shapes, cpu, mems)):
        for hh in range(H):
            sc = scores[a_off:a_off + C].T                           # [G, C]
            assert torch.equal(h[s, hh], O.argmax_first(sc)), "hash is not the first argmax of the scores"
            assert torch.allclose(sc, O.qhash_scores(A[hh:hh + 1], q[s, hh:hh + 1])[0], atol=2e-3, rtol=1e-5)
            a_off += C
        lists = mem.bucket_idx.cpu().long()
        ro, rl = O.hashed_attention_gather(q[s], K, V, lists.reshape(-1), torch.full((H, C), Z), h[s], 128 ** -0.5)
        assert_attn_close(out[s], lse[s], ro, rl, torch.bfloat16, f"decode batch seq {s}")
    # merged with 512 local keys per sequence
    kl = torch.randn(len(shapes), H, 512, d, generator=g).to(torch.bfloat16)
    vl = torch.randn(len(shapes), H, 512, d, generator=g).to(torch.bfloat16)
    mo, ml = batch.attend_with_local(dev(q), dev(kl), dev(vl), 128 ** -0.5)
    for s, ((N, C, Z), (K, V, A), mem) in enumerate(zip(shapes, cpu, mems)):
        lo, ll = O.local_attention(q[s].reshape(1, H * G, 1, d), kl[s:s + 1], vl[s:s + 1], 128 ** -0.5, True)
        eo, el = O.lse_merge_closed_form(lo.reshape(H, G, d).float(), ll.reshape(H, G), out[s].float(), lse[s])
        assert torch.allclose(mo[s].cpu().double(), eo, atol=2e-2, rtol=1e-2)
        assert (ml[s].cpu().double() - el).abs().max().item() < 2e-3
