"""GPU parity checks that separate near-tie effects from wrong results: where a
bf16 score can legitimately reorder two neighbours, the integer part of the result
is compared with a stable sort of the GPU's OWN fp32 scores (bit-exact) and the
floating-point part with the oracle evaluated on those indices; gradients are held
to a per-element bound derived from the terms that are summed, not to a fraction of
the largest gradient."""
import pytest
import torch

from oracle import fm_oracle as O
from tests.util import assert_attn_close, dev, gen, make_attn_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from fast_memory_amd import ops as _ops
    from fast_memory_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return _ops


# ------------------------------------------------------------------ a12, bf16, exactly
def test_compute_centroids_bf16_exact(ops):
    """compute_centroids (memory.py:209-231, 256-258) in bf16, every row: the top-k indices are the first k
    of a stable descending sort of the GPU's own fp32 scores (bit-exact); the centroid is the normalised
    mean of exactly those unit rows (fp64 on the CPU), to bf16 rounding of the result."""
    from fast_memory_amd import compute_centroids
    g = gen(7100)
    H, G, N, d, C, topk = 2, 3, 900, 128, 24, 8
    kq = torch.randn(H * G, N, d, generator=g).to(torch.bfloat16)
    cent = O.init_centroids(C, d, torch.bfloat16)
    kqd, centd = dev(kq, cent)
    A = compute_centroids(kqd, centd, C, G, topk, normalize=True)
    # the steps through the C ABI, one by one
    xn = ops.l2_normalize(kqd, 1e-6)
    ref_xn = O.l2_normalize(kq.float()).to(torch.bfloat16)
    assert (xn.cpu().float() - ref_xn.float()).abs().max().item() <= 2.0 ** -8      # one bf16 step of values <= 1
    Aexp = centd.unsqueeze(0).expand(H * G, -1, -1).contiguous()
    Y = ops.project(Aexp, xn)                                                        # [HG, C, N] fp32
    top = ops.build_index(Aexp, xn, topk)                                            # [HG, C, k]
    assert torch.equal(top.cpu().long(), O.argtopz(Y.cpu(), topk)), "top-k differs from a stable sort of the scores"
    exact = kq.float().double()
    exact = exact / exact.norm(dim=-1, keepdim=True)
    assert torch.allclose(Y.cpu().double(), torch.einsum("cd,hnd->hcn", cent.double(), xn.cpu().double()),
                          atol=1e-4, rtol=1e-5)
    # the mean over the G*k rows of a KV head, from the GPU's normalised rows at the GPU's indices
    rows = xn.cpu().double()[torch.arange(H * G)[:, None, None], top.cpu().long()]   # [HG, C, k, d]
    rows = rows.reshape(H, G, C, topk, d).permute(2, 0, 1, 3, 4).reshape(C, H, G * topk, d)
    want = rows.mean(dim=2)
    want = want / want.norm(dim=-1, keepdim=True)
    got = A.cpu().double()
    assert got.shape == (C, H, d)
    err = (got - want).abs().max().item()
    assert err <= 2.0 ** -8, f"centroid rows off by {err:.3e} given the GPU's own indices"
    # and the composition equals the one call bit for bit
    A2 = ops.topk_mean(xn, top.permute(1, 0, 2).contiguous(), H, G, normalize=True)
    assert torch.equal(A2, A)


# ------------------------------------------------------------------ a15 with the reference's window
@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128)])
def test_attention_hash_with_reference_window(ops, dtype, d):
    """attention_hash with the window the reference hard-codes (triton_kernel.py:283: keys 8192 .. 65535
    kept), against the oracle's composite on the same inputs; lists and hashes against the GPU's own
    scores, so that a bf16 near-tie cannot hide a wrong filter."""
    from fast_memory_amd import attention_hash
    g = gen(7200)
    B, S, N, C, Z = 2, 300, 70000, 12, 700
    q = (torch.randn(B, S, d, generator=g) * 0.7).to(dtype)
    k = (torch.randn(B, N, d, generator=g) * 0.7).to(dtype)
    v = (torch.randn(B, N, d, generator=g) * 0.7).to(dtype)
    A = torch.randn(B, C, d, generator=g).to(dtype)
    lo, hi = 8192, 65536
    qd, kd, vd, Ad = dev(q, k, v, A)
    out, lse = attention_hash(qd, kd, vd, Ad, Z, d ** -0.5, window=(lo, hi))
    lists = O.argtopz(ops.project(Ad, kd).cpu(), Z)                                  # stable sort of the GPU's Y
    assert torch.equal(ops.build_index(Ad, kd, Z).cpu().long(), lists)
    qh, sc = ops.qhash(Ad, qd, return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))
    flat, counts = O.window_filter(lists, lo, hi)                                    # re-based by -lo
    assert int(counts.min()) < Z and int(counts.sum()) > 0                           # the window drops entries
    gflat, gcnt, _ = ops.window_filter(dev(lists.int()), lo, hi)
    assert torch.equal(gcnt.cpu().long(), counts) and torch.equal(gflat.cpu().long()[:int(counts.sum())], flat)
    ro, rl = O.hashed_attention_gather(q, k, v, flat + lo, counts, qh.cpu().long(), d ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, "attention_hash(window)")
    if dtype == torch.float32:
        # no bf16 ties in fp32: the oracle's whole composite, lists and hashes included
        fo, fl, fkh, fqh = O.attention_hash(q, k, v, A, Z, d ** -0.5, window=(lo, hi))
        same = (fqh == qh.cpu().long())
        assert same.float().mean().item() > 0.99
        assert torch.allclose(out.cpu()[same], fo[same], atol=1e-4, rtol=1e-4)


# ------------------------------------------------------------------ f1: per-element gradient bounds
def _grads_with_bounds(q, k, v, kh, cnt, qh, out, lse, dout, sm):
    """fp64 gradients of the gathered attention (the formulas of memory.py:166-206 restricted to each query's
    bucket) and, beside each, the sum of the absolute values of the terms it adds up: a result computed
    with terms rounded to relative eps is within eps times that sum."""
    H, Sq, d = q.shape
    N = k.shape[1]
    off = O.bucket_offsets(cnt)
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    dq, dk, dv = z(H, Sq, d), z(H, N, d), z(H, N, d)
    bq, bk, bv = z(H, Sq, d), z(H, N, d), z(H, N, d)
    q, k, v, out, dout, lse = (t.double() for t in (q, k, v, out, dout, lse))
    for h in range(H):
        for b in range(cnt.shape[1]):
            c = int(cnt[h, b])
            sel = (qh[h] == b).nonzero().flatten()
            if c == 0 or sel.numel() == 0:
                continue
            idx = kh[int(off[h, b]):int(off[h, b]) + c].long()
            kk, vv, qq, do = k[h, idx], v[h, idx], q[h, sel], dout[h, sel]
            p = torch.exp(qq @ kk.T * sm - lse[h, sel][:, None])                     # [nq, c]
            dp = do @ vv.T
            D = (do * out[h, sel]).sum(-1, keepdim=True)
            ds = p * (dp - D)
            dq[h, sel] = sm * ds @ kk
            bq[h, sel] = sm * ds.abs() @ kk.abs()
            dk[h].index_add_(0, idx, sm * ds.T @ qq)
            bk[h].index_add_(0, idx, sm * ds.abs().T @ qq.abs())
            dv[h].index_add_(0, idx, p.T @ do)
            bv[h].index_add_(0, idx, p.T @ do.abs())
    return (dq, dk, dv), (bq, bk, bv)


def _worst_ratio(got, ref, bound, out_eps):
    """max over elements of |got - ref| / (2^-9 * bound + out_eps * |ref| + 1e-7): 1 means every summed term
    was off by half a bf16 unit in the same direction."""
    got = got.float().cpu().double()
    return ((got - ref).abs() / (2.0 ** -9 * bound + out_eps * ref.abs() + 1e-7)).max().item()


@pytest.mark.parametrize("B,S,N,C,Z", [(2, 200, 2000, 12, 150), (1, 600, 900, 3, 333)])
def test_bf16_backward_within_per_element_bounds(ops, B, S, N, C, Z):
    """bf16 MFMA backward, atomic and staged forms: p and dS are rounded to bf16 before the MFMAs that sum
    them (relative 2^-9 per term), dq is stored in bf16; everything else is fp32.  The error of every
    gradient element must stay within a small multiple of 2^-9 times the sum of |terms| of THAT element
    (the staged form adds one bf16 rounding of each bucket's partial row)."""
    from fast_memory_amd import attention_hash_varlen
    d, sm = 128, 128 ** -0.5
    q, k, v, kh, cnt, qh = make_attn_case(7300 + S, B, S, N, C, Z, d, torch.bfloat16, window="ref", std=0.7)
    dout = (torch.randn(B, S, d, generator=gen(7301)) * 0.5).to(torch.bfloat16)
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(qd, kd, vd, khd, cntd, qhd, sm)
    lists, counts = khd.int().contiguous(), cntd.int().contiguous()
    off = ops.bucket_offsets(counts)
    groups = ops.group_queries(qhd.int().contiguous(), C)
    (rq, rk, rv), (bq, bk, bv) = _grads_with_bounds(q, k, v, kh, cnt, qh, out.cpu(), lse.cpu(), dout, sm)
    dq, dk, dv = ops.hash_attn_bwd(qd, kd, vd, lists, off, counts, groups, out, lse, dev(dout), sm)
    r = (_worst_ratio(dq, rq, bq, 2.0 ** -8), _worst_ratio(dk, rk, bk, 0.0), _worst_ratio(dv, rv, bv, 0.0))
    print(f"atomic backward, worst error / bound: dq {r[0]:.2f} dk {r[1]:.2f} dv {r[2]:.2f}", flush=True)
    assert max(r) <= 3.0, r
    inv = ops.inverse_index(lists, off, counts, N)
    dq, dk, dv = ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm)
    # partial rows are bf16: 2^-9 of each bucket's contribution, which the term sums bound as well
    r = (_worst_ratio(dq, rq, bq, 2.0 ** -8), _worst_ratio(dk, rk, 2 * bk, 0.0), _worst_ratio(dv, rv, 2 * bv, 0.0))
    print(f"staged backward, worst error / bound: dq {r[0]:.2f} dk {r[1]:.2f} dv {r[2]:.2f}", flush=True)
    assert max(r) <= 3.0, r


# ------------------------------------------------------------------ ring backward on a window that drops entries
@pytest.mark.parametrize("rank", [0, 1])
def test_ring_backward_bf16_window_drops_entries(ops, rank):
    """ring_attention_masked_backward (memory.py:166-206) in the production dtype with more queries than
    buckets, on one of two key windows: the window filter's output buffer is longer than the surviving
    lists, and the staged backward (taken by default for this shape) must read only the survivors.
    Against the oracle's dense-masked restatement and against the atomic form."""
    from fast_memory_amd import ring_attention_masked_backward, ring_attention_masked_forward
    from fast_memory_amd.hash_attention import attention_hash_varlen_backward
    g = gen(7400)
    C, H, G, S, N, Z, d, world = 8, 2, 2, 40, 300, 96, 128, 2
    sm = d ** -0.5
    q = (torch.randn(1, H * G, S, d, generator=g) * 0.7).to(torch.bfloat16)
    k = (torch.randn(1, H, N, d, generator=g) * 0.7).to(torch.bfloat16)
    v = (torch.randn(1, H, N, d, generator=g) * 0.7).to(torch.bfloat16)
    w = (torch.randn(1, H * G, S, d, generator=g) * 0.5).to(torch.bfloat16)
    kh = torch.stack([torch.stack([torch.randperm(world * N, generator=g)[:Z] for _ in range(H)]) for _ in range(C)])
    qh = torch.randint(0, C, (H, G, S), generator=g)
    assert G * S >= C                                                   # the shape that takes the staged form
    out, lse = ring_attention_masked_forward(*dev(kh, qh, q, k, v), sm, rank)
    dq, dk, dv = ring_attention_masked_backward(*dev(kh, qh), torch.arange(H), dev(w), dev(q), dev(k), dev(v),
                                                out, lse, sm, rank)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape and dk.dtype == torch.bfloat16
    rq, rk, rv = O.ring_attention_masked_backward_ref(kh, qh, w.float(), q.float(), k.float(), v.float(),
                                                      out.float().cpu(), lse.cpu(), sm, rank)
    for got, ref, name in ((dq, rq, "dq"), (dk, rk, "dk"), (dv, rv, "dv")):
        got, ref = got.float().cpu().double(), ref.double()
        assert torch.allclose(got, ref, atol=2e-2 * max(1.0, ref.abs().max().item()), rtol=2e-2), \
            f"rank {rank} {name}: max err {(got - ref).abs().max().item():.3e}"
    # the same call with the atomic form
    khw = kh.permute(1, 0, 2).to(torch.int32).contiguous()
    flat, counts, _ = ops.window_filter(dev(khw), rank * N, (rank + 1) * N)
    assert flat.numel() > int(counts.sum())                             # the buffer has an unused tail
    args = (dev(w).reshape(H, -1, d).contiguous(), dev(q).reshape(H, -1, d).contiguous(), dev(k)[0], dev(v)[0],
            out.reshape(H, -1, d), lse.reshape(H, -1), flat, counts, dev(qh).reshape(H, -1), sm)
    s_dq, s_dk, s_dv = attention_hash_varlen_backward(*args, staged=True)
    a_dq, a_dk, a_dv = attention_hash_varlen_backward(*args, staged=False)
    for a, b, name in ((s_dq, a_dq, "dq"), (s_dk, a_dk, "dk"), (s_dv, a_dv, "dv")):
        a, b = a.float(), b.float()
        assert torch.allclose(a, b, atol=1e-2 * max(1.0, b.abs().max().item()), rtol=1e-2), name


def test_backward_with_every_entry_outside_the_window(ops):
    """A window that keeps nothing: every bucket is empty, the gradients are zero, nothing is staged."""
    from fast_memory_amd import ring_attention_masked_backward, ring_attention_masked_forward
    g = gen(7500)
    C, H, G, S, N, Z, d = 4, 1, 2, 8, 64, 16, 128
    q = torch.randn(1, H * G, S, d, generator=g).to(torch.bfloat16)
    k = torch.randn(1, H, N, d, generator=g).to(torch.bfloat16)
    v = torch.randn(1, H, N, d, generator=g).to(torch.bfloat16)
    kh = torch.stack([torch.stack([torch.randperm(N, generator=g)[:Z] for _ in range(H)]) for _ in range(C)])
    qh = torch.randint(0, C, (H, G, S), generator=g)
    out, lse = ring_attention_masked_forward(*dev(kh, qh, q, k, v), 0.1, 3)          # window [3N, 4N): no entry
    assert bool((out == 0).all()) and bool((lse < -1e30).all())
    dq, dk, dv = ring_attention_masked_backward(*dev(kh, qh), torch.arange(H), dev(q), dev(q), dev(k), dev(v),
                                                out, lse, 0.1, 3)
    assert bool((dq == 0).all()) and bool((dk == 0).all()) and bool((dv == 0).all())


# ------------------------------------------------------------------ a5: hashes outside [0, C)
@pytest.mark.parametrize("dtype,d", [(torch.float32, 64), (torch.bfloat16, 128)])
def test_out_of_range_query_hash_is_an_empty_bucket(ops, dtype, d):
    """The reference would raise on a query hash outside [0, C) (an index error at triton_kernel.py:84);
    the one-call operator defines it: such a query gets the result of an empty bucket, every other query
    is unaffected, and the grouping counts it nowhere."""
    from fast_memory_amd import attention_hash_varlen
    q, k, v, kh, cnt, qh = make_attn_case(7600, 2, 90, 500, 5, 40, d, dtype, window="all")
    bad = torch.zeros_like(qh, dtype=torch.bool)
    bad[0, 3], bad[0, 50], bad[1, 89] = True, True, True
    qh_bad = qh.clone()
    qh_bad[0, 3], qh_bad[0, 50], qh_bad[1, 89] = -1, 5, 1 << 20
    out, lse = attention_hash_varlen(*dev(q, k, v, kh, cnt, qh_bad), 0.2)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 0.2)
    assert bool((out[dev(bad)] == 0).all()) and bool((lse[dev(bad)] < -1e30).all())
    good = ~bad
    assert_attn_close(out[dev(good)][None], lse[dev(good)][None], ro[good][None], rl[good][None], dtype, "others")
    groups = ops.group_queries(dev(qh_bad.int()), 5)
    assert torch.equal(groups.bin_count.cpu().long(),
                       torch.stack([torch.bincount(qh[b][good[b]], minlength=5) for b in range(2)]))
    # the grouped queries fill the first slots of q_perm, the three without a bucket the last ones, coded
    # as -(flat query index) - 1
    tail = sorted((-groups.q_perm.reshape(-1)[-3:].cpu().long() - 1).tolist())
    assert tail == [3, 50, 90 + 89]
    # every forward entry defines those rows, not only the one-call operator: poison the outputs' memory
    # first (the caching allocator hands the same blocks out again)
    off = ops.bucket_offsets(dev(cnt.int()))
    for _ in range(2):
        junk = torch.full((2, 90, d), float("nan"), dtype=dtype, device="cuda")
        junk_l = torch.full((2, 90), float("nan"), device="cuda")
        del junk, junk_l
        o2, l2 = ops.hash_attn_fwd(*dev(q, k, v, kh.int()), off, dev(cnt.int()), groups, 0.2)
        assert torch.equal(o2, out) and torch.equal(l2, lse)
    # ... and so does the backward: dq = 0 for them, the other gradients as without them
    from fast_memory_amd import attention_hash_varlen_op
    g = gen(7601)
    w = (torch.randn(2, 90, d, generator=g) * 0.5).to(dtype)
    w0 = w.clone()
    w0[bad] = 0                                            # "good" run: the three queries hashed, their d_out zero
    grads = {}
    for name, hashes, wt in (("bad", qh_bad, w), ("good", qh, w0)):
        qd, kd, vd = (t.requires_grad_(True) for t in dev(q, k, v))
        junk = torch.full((2, 90, d), float("nan"), dtype=dtype, device="cuda")
        del junk
        o3, _ = attention_hash_varlen_op(qd, kd, vd, *dev(kh, cnt, hashes), 0.2)
        (o3.float() * dev(wt).float()).sum().backward()
        grads[name] = (qd.grad, kd.grad, vd.grad)
    assert bool((grads["bad"][0][dev(bad)] == 0).all()), "dq of a query without a bucket"
    assert torch.equal(grads["bad"][0][dev(good)], grads["good"][0][dev(good)])
    # dk / dv: a query with zero d_out contributes nothing, so the two runs agree up to the order of the
    # fp32 atomic adds
    for j in (1, 2):
        a, b = grads["bad"][j].float(), grads["good"][j].float()
        assert bool(torch.isfinite(a).all())
        # (bf16 takes the form without atomics, whose per-bucket partial rows are bf16 sums over query tiles:
        # three queries fewer in a row move the tile boundaries, and with them those roundings)
        if dtype == torch.float32:
            assert torch.allclose(a, b, atol=1e-5 * max(1.0, b.abs().max().item()), rtol=1e-4)
        else:
            assert (a - b).abs().max().item() <= 2e-2 * b.abs().max().item()


# ------------------------------------------------------------------ a2 in the fused build: ties and long runs
@pytest.mark.parametrize("copies", [3, 40, 700])
def test_fused_build_with_duplicated_keys(ops, copies):
    """The selection of the fused build places every candidate by counting the larger ones in its value
    bin, and hands rows with very long runs of (nearly) equal values to the radix select and the sorting
    network.  Keys repeated `copies` times give runs of exactly equal projections -- short runs stay in
    the bins (ties by ascending index), 700 copies exceed what a bin takes -- and in every case the lists
    must equal the stable descending sort of the GPU's own Y and those of the unfused build."""
    g = gen(7700 + copies)
    H, C, N, d, Z = 1, 24, 70000, 128, 2048
    base = (torch.randn(H, N // copies + 1, d, generator=g) * 0.5)
    K = base.repeat_interleave(copies, dim=1)[:, :N]
    perm = torch.randperm(N, generator=g)
    K = K[:, perm].contiguous().to(torch.bfloat16)                 # equal keys scattered over the index range
    A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
    Ad, Kd = dev(A, K)
    fused, fv = ops.build_index(Ad, Kd, Z, fused=True, return_values=True)
    assert ops.last_build_info["path"] == "fused" and ops.last_build_info["rows_unresolved"] == 0
    Y = ops.project(Ad, Kd).cpu()
    ref = torch.sort(Y + 0.0, dim=-1, descending=True, stable=True)
    assert torch.equal(fused.cpu().long(), ref.indices[..., :Z]), "lists differ from the stable sort"
    assert torch.equal(fv.cpu(), ref.values[..., :Z])
    assert torch.equal(fused, ops.build_index(Ad, Kd, Z, fused=False))


def test_staged_backward_with_thousands_of_queries_in_one_bucket(ops):
    """A heavily skewed hash: 2300 of a row's 2400 queries fall into one bucket.  Only the first 256 queries of
    a bucket go through its bf16 partial rows (every further pass would round them again); the rest is added
    with fp32 atomics.  dK and dV must stay within the per-element bound of the atomic form -- with all
    queries going through the partial rows the error grows with the number of passes."""
    from fast_memory_amd import attention_hash_varlen
    B, S, N, C, Z, d, sm = 1, 2400, 1200, 4, 300, 128, 128 ** -0.5
    q, k, v, kh, cnt, qh = make_attn_case(7800, B, S, N, C, Z, d, torch.bfloat16, window="all", std=0.7)
    qh[0, :2300] = 1
    dout = (torch.randn(B, S, d, generator=gen(7801)) * 0.5).to(torch.bfloat16)
    qd, kd, vd, khd, cntd, qhd = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(qd, kd, vd, khd, cntd, qhd, sm)
    lists, counts = khd.int().contiguous(), cntd.int().contiguous()
    off = ops.bucket_offsets(counts)
    groups = ops.group_queries(qhd.int().contiguous(), C)
    inv = ops.inverse_index(lists, off, counts, N)
    (rq, rk, rv), (bq, bk, bv) = _grads_with_bounds(q, k, v, kh, cnt, qh, out.cpu(), lse.cpu(), dout, sm)
    dq, dk, dv = ops.hash_attn_bwd_staged(qd, kd, vd, lists, off, counts, groups, inv, out, lse, dev(dout), sm)
    r = (_worst_ratio(dq, rq, bq, 2.0 ** -8), _worst_ratio(dk, rk, 2 * bk, 0.0), _worst_ratio(dv, rv, 2 * bv, 0.0))
    print(f"staged backward, 2300 queries in one bucket, worst error / bound: dq {r[0]:.2f} dk {r[1]:.2f} dv {r[2]:.2f}",
          flush=True)
    assert max(r) <= 3.0, r
    dq2, dk2, dv2 = ops.hash_attn_bwd(qd, kd, vd, lists, off, counts, groups, out, lse, dev(dout), sm)
    assert torch.equal(dq.view(torch.int16)[0, 2300:], dq2.view(torch.int16)[0, 2300:])      # same tile code
    assert torch.allclose(dk, dk2, atol=2e-2 * float(dk2.abs().max()), rtol=2e-2)
