"""Seeded random extents through the one-call operator, its backward, the hash and the index build, each against
the oracle: extents that no hand-picked case names (odd sizes, lists of one key, more buckets than queries, a
single query, head dimensions between the MFMA kernels' own)."""
import random

import pytest
import torch

from oracle import fm_oracle as O
from tests.util import assert_attn_close, dev, gen, make_attn_case

pytestmark = pytest.mark.gpu

_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def _cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["f32", "bf16", "bf16", "f16"])
        d = rnd.choice([16, 32, 48, 64, 128, 128, 256] if dt != "f32" else [8, 16, 40, 64, 128])
        B = rnd.randint(1, 3)
        N = rnd.choice([1, 7, 63, 64, 65, 200, 1000, 2500])
        C = rnd.choice([1, 2, 5, 16, 33])
        Z = rnd.randint(1, min(N, 300))
        S = rnd.choice([1, 2, 15, 16, 17, 64, 65, 130, 300])
        out.append(pytest.param(dt, B, S, N, C, Z, d, 4000 + i, id=f"{dt}-B{B}-S{S}-N{N}-C{C}-Z{Z}-d{d}"))
    return out


@pytest.mark.parametrize("dt,B,S,N,C,Z,d,seed", _cases(60, 20260))
def test_operator_forward_and_backward_random_extents(dt, B, S, N, C, Z, d, seed):
    from fast_memory_amd import attention_hash_varlen, attention_hash_varlen_backward
    dtype = _DT[dt]
    q, k, v, kh, cnt, qh = make_attn_case(seed, B, S, N, C, Z, d, dtype, window="ref", std=0.6)
    sm = d ** -0.5
    args = dev(q, k, v, kh, cnt, qh)
    out, lse = attention_hash_varlen(*args, sm)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, sm)
    assert_attn_close(out, lse, ro, rl, dtype, "forward")
    dout = (torch.randn(B, S, d, generator=gen(seed + 1)) * 0.5).to(dtype)
    dq, dk, dv = attention_hash_varlen_backward(dev(dout), args[0], args[1], args[2], out, lse, args[3], args[4],
                                                args[5], sm)
    rq, rk, rv = O.hashed_attention_backward_gather(q.float(), k.float(), v.float(), kh, cnt, qh, out.float().cpu(),
                                                    lse.cpu(), dout.float(), sm)
    for got, ref, name in ((dq, rq, "dq"), (dk, rk, "dk"), (dv, rv, "dv")):
        got, ref = got.float().cpu().double(), ref.double()
        tol = 1e-4 if dtype == torch.float32 else 2e-2
        assert torch.allclose(got, ref, atol=tol * max(1.0, ref.abs().max().item()), rtol=tol), \
            f"{name}: {(got - ref).abs().max().item():.3e} (ref max {ref.abs().max().item():.3e})"


def _build_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["f32", "bf16", "f16"])
        d = rnd.choice([16, 64, 128, 128, 256])
        H = rnd.randint(1, 3)
        N = rnd.choice([100, 1000, 4097, 70001, 90000])
        C = rnd.choice([1, 3, 17, 64, 130])
        Z = rnd.choice([1, 5, 64, 100, 1000])
        Z = min(Z, N)
        S = rnd.choice([1, 33, 500])
        out.append(pytest.param(dt, H, N, C, Z, S, d, 5000 + i, id=f"{dt}-H{H}-N{N}-C{C}-Z{Z}-S{S}-d{d}"))
    return out


@pytest.mark.parametrize("dt,H,N,C,Z,S,d,seed", _build_cases(30, 20261))
def test_build_and_hash_random_extents(dt, H, N, C, Z, S, d, seed):
    """Lists and hashes bit-exact against the oracle on the device's own fp32 scores (whichever build path the
    extents take: fused for bf16 / fp16 at d = 128 with 16 384 keys or more and enough rows, chunked otherwise)."""
    from fast_memory_amd import ops
    dtype = _DT[dt]
    g = gen(seed)
    K = (torch.randn(H, N, d, generator=g) * 0.5).to(dtype)
    A = torch.randn(H, C, d, generator=g).to(dtype)
    Q = (torch.randn(H, S, d, generator=g) * 0.5).to(dtype)
    Ad, Kd, Qd = dev(A, K, Q)
    lists = ops.build_index(Ad, Kd, Z)
    Y = ops.project(Ad, Kd).cpu()
    assert torch.equal(lists.cpu().long(), O.argtopz(Y, Z))
    qh, sc = ops.qhash(Ad, Qd, return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))


def _local_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["f32", "bf16", "f16"])
        d = rnd.choice([32, 64, 128, 256] if dt != "f32" else [16, 64, 128])
        H, G = rnd.randint(1, 2), rnd.choice([1, 2, 3, 8])
        S = rnd.choice([1, 2, 31, 32, 33, 127, 128, 129, 300])
        L = rnd.choice([1, 5, 63, 64, 65, 200, 513])
        causal = rnd.random() < 0.7
        out.append(pytest.param(dt, H, G, S, L, d, causal, 6000 + i, id=f"{dt}-H{H}-G{G}-S{S}-L{L}-d{d}-{'causal' if causal else 'full'}"))
    return out


@pytest.mark.parametrize("dt,H,G,S,L,d,causal,seed", _local_cases(36, 20262))
def test_local_attention_random_extents(dt, H, G, S, L, d, causal, seed):
    """The dense local attention (more queries than keys included: with the causal mask aligned bottom-right
    the first S - L queries then see nothing and get out = 0, lse = -FLT_MAX)."""
    from fast_memory_amd import ops
    dtype = _DT[dt]
    g = gen(seed)
    q = torch.randn(1, H * G, S, d, generator=g).to(dtype)
    k = torch.randn(1, H, L, d, generator=g).to(dtype)
    v = torch.randn(1, H, L, d, generator=g).to(dtype)
    out, lse = ops.local_attn_fwd(dev(q[0]), dev(k[0]), dev(v[0]), d ** -0.5, causal)
    ro, rl = O.local_attention(q, k, v, d ** -0.5, causal)
    assert_attn_close(out, lse, ro[0], rl[0], dtype, "local")


def _memory_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["f32", "bf16", "bf16", "f16"])
        d = rnd.choice([64, 128, 128] if dt != "f32" else [16, 64])
        H, G = rnd.randint(1, 2), rnd.choice([1, 2, 4])
        N0 = rnd.choice([10, 300, 2000, 66000])
        M = rnd.choice([1, 7, 100, 700])
        C = rnd.choice([1, 4, 13, 40])
        Z = rnd.choice([1, 16, 100, 512])
        S = rnd.choice([1, 5, 40])
        L = rnd.choice([1, 40, 70])
        out.append(pytest.param(dt, H, G, N0, M, C, Z, S, L, d, 7000 + i,
                                id=f"{dt}-H{H}-G{G}-N{N0}+{M}-C{C}-Z{Z}-S{S}-L{L}-d{d}"))
    return out


@pytest.mark.parametrize("dt,H,G,N0,M,C,Z,S,L,d,seed", _memory_cases(24, 20263))
def test_memory_build_append_attend_random_extents(dt, H, G, N0, M, C, Z, S, L, d, seed):
    """A memory through its life: built (lists shorter than Z while it holds fewer than Z keys), extended, asked
    with local keys -- the lists against the oracle's arg-top-Z of the device's scores, the merged attention
    against one softmax over the hashed bucket's keys and the visible local keys."""
    from fast_memory_amd import Memory, ops
    dtype = _DT[dt]
    g = gen(seed)
    K = (torch.randn(H, N0 + M, d, generator=g) * 0.5).to(dtype)
    V = (torch.randn(H, N0 + M, d, generator=g) * 0.5).to(dtype)
    A = torch.randn(H, C, d, generator=g).to(dtype)
    q = (torch.randn(H, G * S, d, generator=g) * 0.5).to(dtype)
    kl = (torch.randn(H, L, d, generator=g) * 0.5).to(dtype)
    vl = (torch.randn(H, L, d, generator=g) * 0.5).to(dtype)
    Kd, Vd, Ad, qd = dev(K, V, A, q)
    mem = Memory.build(Kd[:, :N0].contiguous(), Vd[:, :N0].contiguous(), Ad, Z, keep_values=True)
    mem.append(Kd[:, N0:].contiguous(), Vd[:, N0:].contiguous())
    N = N0 + M
    Zl = min(Z, N)                                            # a memory of fewer than Z keys lists them all
    Y = ops.project(Ad, Kd).cpu()
    want = O.argtopz(Y, Zl)
    cnt = mem.bucket_cnt.cpu()
    assert (cnt == Zl).all()
    assert torch.equal(mem.bucket_idx.cpu().long()[..., :Zl], want)
    sm = d ** -0.5
    out, lse = mem.attend_with_local(qd, *dev(kl, vl), sm, n_groups=G, causal=True)
    qh = mem.hash(qd).cpu().long()
    o64, l64 = out.cpu().double(), lse.cpu().double()
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for h in range(H):
        for i in range(0, G * S, max(1, (G * S) // 7)):
            t = i % S                                          # token of query i inside its query head
            vis = min(L, max(0, t + (L - S) + 1))              # local keys it sees (mask aligned bottom-right)
            idx = want[h, qh[h, i]]
            kk = torch.cat([K[h, idx], kl[h, :vis]]).double()
            vv = torch.cat([V[h, idx], vl[h, :vis]]).double()
            s = kk @ q[h, i].double() * sm
            assert abs(torch.logsumexp(s, 0).item() - l64[h, i].item()) < 1e-3
            assert torch.allclose(torch.softmax(s, 0) @ vv, o64[h, i], atol=tol, rtol=tol)


@pytest.mark.parametrize("seed", [8001, 8002, 8003, 8004, 8005, 8006])
def test_decode_batch_random_extents(seed):
    """Batched decode over memories of random lengths, bucket counts and list lengths (one token per query
    head), hashes against the first argmax of the returned scores, attention against the oracle."""
    from fast_memory_amd import Memory, MemoryBatch
    rnd = random.Random(seed)
    g = gen(seed)
    H, G, d = rnd.randint(1, 3), rnd.choice([1, 2, 4, 8, 16]), 128
    n_seq = rnd.randint(1, 6)
    shapes = []
    for _ in range(n_seq):
        N = rnd.choice([1, 50, 700, 3000, 9000])
        C = rnd.choice([1, 3, 26, 64, 95])
        shapes.append((N, C, rnd.randint(1, min(N, 400))))
    mems, cpu = [], []
    for N, C, Z in shapes:
        K = torch.randn(H, N, d, generator=g).to(torch.bfloat16)
        V = torch.randn(H, N, d, generator=g).to(torch.bfloat16)
        A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
        mems.append(Memory.build(*dev(K, V, A), Z))
        cpu.append((K, V, A))
    batch = MemoryBatch(mems)
    q = (torch.randn(n_seq, H, G, d, generator=g) * 1.5).to(torch.bfloat16)
    out, lse, h, scores = batch.attend(dev(q), d ** -0.5, return_scores=True)
    out, lse, h, scores = out.cpu(), lse.cpu(), h.cpu().long(), scores.cpu()
    a_off = 0
    for s, ((N, C, Z), (K, V, A), mem) in enumerate(zip(shapes, cpu, mems)):
        for hh in range(H):
            sc = scores[a_off:a_off + C].T
            assert torch.equal(h[s, hh], O.argmax_first(sc)), f"seq {s} head {hh}: hash"
            a_off += C
        lists = mem.bucket_idx.cpu().long()
        ro, rl = O.hashed_attention_gather(q[s], K, V, lists.reshape(-1), torch.full((H, C), Z), h[s], d ** -0.5)
        assert_attn_close(out[s], lse[s], ro, rl, torch.bfloat16, f"decode batch seq {s} {shapes[s]}")


def _window_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["f32", "bf16", "f16"])
        d = rnd.choice([64, 128] if dt != "f32" else [16, 64])
        B = rnd.randint(1, 2)
        N = rnd.choice([500, 3000, 70000])
        C = rnd.choice([2, 9, 30])
        Z = rnd.choice([8, 64, 300])
        S = rnd.choice([3, 50, 400])
        lo = rnd.choice([0, 0, N // 3, N - 5])
        hi = rnd.choice([N, lo + 1, lo + max(1, (N - lo) // 2), lo])       # the last: an empty window
        out.append(pytest.param(dt, B, S, N, C, Z, d, lo, hi, 9000 + i, id=f"{dt}-B{B}-S{S}-N{N}-C{C}-Z{Z}-d{d}-w{lo}:{hi}"))
    return out


@pytest.mark.parametrize("dt,B,S,N,C,Z,d,lo,hi,seed", _window_cases(20, 20264))
def test_attention_hash_with_window_random_extents(dt, B, S, N, C, Z, d, lo, hi, seed):
    """The composite (build + hash + attention, triton_kernel.py:275-286) with a window of key indices as the
    reference hard-codes one (triton_kernel.py:283), including windows no listed key falls into."""
    from fast_memory_amd import attention_hash, ops
    dtype = _DT[dt]
    g = gen(seed)
    q = (torch.randn(B, S, d, generator=g) * 0.5).to(dtype)
    k = (torch.randn(B, N, d, generator=g) * 0.5).to(dtype)
    v = (torch.randn(B, N, d, generator=g) * 0.5).to(dtype)
    cen = torch.randn(B, C, d, generator=g).to(dtype)
    qd, kd, vd, cd = dev(q, k, v, cen)
    sm = d ** -0.5
    out, lse = attention_hash(qd, kd, vd, cd, Z, sm, window=(lo, hi))
    lists = O.argtopz(ops.project(cd, kd).cpu(), Z)
    qh, sc = ops.qhash(cd, qd, return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))
    mask = (lists >= lo) & (lists < hi)
    ro, rl = O.hashed_attention_gather(q, k, v, lists[mask], mask.sum(-1), qh.cpu().long(), sm)
    assert_attn_close(out, lse, ro, rl, dtype, "attention_hash with a window")


def _dispatch_cases(n, seed):
    rnd = random.Random(seed)
    out = []
    for i in range(n):
        dt = rnd.choice(["bf16", "f16"])
        d = rnd.choice([64, 128, 128, 128, 256])
        B = rnd.randint(1, 3)
        N = rnd.choice([5000, 40000, 300000])
        C = rnd.choice([1, 8, 64, 700])
        Z = rnd.choice([1, 64, 700, 3000])
        S = rnd.choice([10, 700, 9000])
        skew = rnd.random() < 0.3
        out.append(pytest.param(dt, B, S, N, C, Z, d, skew, 9500 + i, id=f"{dt}-B{B}-S{S}-N{N}-C{C}-Z{Z}-d{d}{'-skew' if skew else ''}"))
    return out


@pytest.mark.parametrize("dt,B,S,N,C,Z,d,skew,seed", _dispatch_cases(48, 20265))
def test_mfma_kernels_against_generic_random_extents(dt, B, S, N, C, Z, d, skew, seed):
    """Whatever kernel the dispatch takes for the extents (rows gathered into registers, staged in LDS, loaded
    straight into LDS; one launch or one per row; forward and backward) against the generic kernels on the same
    device inputs -- at sizes the CPU oracle would take minutes for.  ``skew``: a third of the queries in one
    bucket (several work items and workgroups for it)."""
    from fast_memory_amd import attention_hash_varlen, attention_hash_varlen_backward, ops
    dtype = _DT[dt]
    g = torch.Generator(device="cuda").manual_seed(seed)
    mk = lambda *s: (torch.randn(*s, generator=g, device="cuda") * 0.6).to(dtype)
    q, k, v, dout = mk(B, S, d), mk(B, N, d), mk(B, N, d), mk(B, S, d)
    lists = torch.randint(0, N, (B, C, Z), generator=g, device="cuda", dtype=torch.int32)
    cnt = torch.randint(0, Z + 1, (B, C), generator=g, device="cuda", dtype=torch.int32)       # ragged, some empty
    keep = torch.arange(Z, device="cuda")[None, None, :] < cnt[..., None]
    flat = lists[keep].contiguous()
    qh = torch.randint(0, C, (B, S), generator=g, device="cuda", dtype=torch.int32)
    if skew:
        qh[:, : S // 3] = C // 2
    sm = d ** -0.5
    run = lambda: attention_hash_varlen(q, k, v, flat, cnt, qh, sm, lse_dtype=torch.float32)
    bwd = lambda o, l: attention_hash_varlen_backward(dout, q, k, v, o, l, flat, cnt, qh, sm)
    o1, l1 = run()
    g1 = bwd(o1, l1)
    ops.force_generic_kernels(True)
    try:
        o2, l2 = run()
        g2 = bwd(o1, l1)                                                   # the same out / lse into both backwards
    finally:
        ops.force_generic_kernels(False)
    empty = l2 < -1e30
    assert torch.equal(l1 < -1e30, empty)
    assert torch.allclose(o1.float(), o2.float(), atol=2e-2, rtol=1e-2)
    assert (l1[~empty] - l2[~empty]).abs().max().item() < 1e-3 if (~empty).any() else True
    for a, b, name in zip(g1, g2, ("dq", "dk", "dv")):
        a, b = a.float(), b.float()
        assert torch.allclose(a, b, atol=2e-2 * max(1.0, b.abs().max().item()), rtol=2e-2), \
            f"{name}: {(a - b).abs().max().item():.3e} vs max {b.abs().max().item():.3e}"


def _forced_cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        which = ("wave", "wave-per-row", "ring", "ring-per-row", "staged", "staged-pairs")[i % 6]
        dt = rng.choice(["bf16", "f16"])
        B = rng.choice([1, 2, 3])
        N = rng.randint(40, 6000)
        C = rng.randint(1, 48)
        Z = rng.randint(1, min(N, 700))
        S = rng.randint(1, 1500)
        out.append(pytest.param(which, dt, B, S, N, C, Z, rng.random() < 0.4, seed + i, id=f"{i}-{which}-{dt}-B{B}-S{S}-N{N}-C{C}-Z{Z}"))
    return out


@pytest.mark.parametrize("which,dt,B,S,N,C,Z,skew,seed", _forced_cases(48, 20266))
def test_forced_forward_kernels_against_generic_and_themselves_random_extents(which, dt, B, S, N, C, Z, skew, seed):
    """Each d = 128 forward kernel forced on shapes dispatch would never give it (a wave per work item on short
    lists and on items of 49-64 queries, which it sweeps twice; three items per workgroup on single-query
    buckets, ...): against the generic kernel on the same device inputs, and twice in a row with the same bits
    (a result may not depend on timing)."""
    from fast_memory_amd import attention_hash_varlen, ops
    dtype = _DT[dt]
    g = torch.Generator(device="cuda").manual_seed(seed)
    mk = lambda *s: (torch.randn(*s, generator=g, device="cuda") * 0.6).to(dtype)
    q, k, v = mk(B, S, 128), mk(B, N, 128), mk(B, N, 128)
    lists = torch.randint(0, N, (B, C, Z), generator=g, device="cuda", dtype=torch.int32).sort(-1).values
    cnt = torch.randint(0, Z + 1, (B, C), generator=g, device="cuda", dtype=torch.int32)       # ragged, some empty
    keep = torch.arange(Z, device="cuda")[None, None, :] < cnt[..., None]
    flat = lists[keep].contiguous()
    qh = torch.randint(0, C, (B, S), generator=g, device="cuda", dtype=torch.int32)
    if skew:
        qh[:, : S // 3] = C // 2
    run = lambda: attention_hash_varlen(q, k, v, flat, cnt, qh, 128 ** -0.5, lse_dtype=torch.float32)
    ops.grouped_forward_kernel(which)
    try:
        o1, l1 = run()
        o1b, l1b = run()
    finally:
        ops.grouped_forward_kernel(None)
    assert torch.equal(o1, o1b) and torch.equal(l1, l1b), "two runs of one kernel on the same inputs differ"
    ops.force_generic_kernels(True)
    try:
        o2, l2 = run()
    finally:
        ops.force_generic_kernels(False)
    empty = l2 < -1e30
    assert torch.equal(l1 < -1e30, empty)
    assert torch.allclose(o1.float(), o2.float(), atol=2e-2, rtol=1e-2)
    assert (l1[~empty] - l2[~empty]).abs().max().item() < 1e-3 if (~empty).any() else True


@pytest.mark.parametrize("C,S", [(1025, 5000), (1500, 9000), (2048, 40000), (2600, 12000), (4200, 30000)])
def test_wave_per_row_takes_every_item_once_in_the_paired_order(C, S):
    """Rows of more than 1024 work items: a launch of the wave-per-item kernel takes them in an order of its own
    (heavy and light items paired), chunk by chunk of 2048 slots -- a last chunk of any length, items of one to
    four tiles of queries and items swept twice.  Against the generic kernel, and bit for bit against the
    single launch over all rows, which takes the items in the order they come."""
    from fast_memory_amd import attention_hash_varlen, ops
    B, N, Z = 2, 4096, 48
    g = torch.Generator(device="cuda").manual_seed(C * 7 + S)
    mk = lambda *s: (torch.randn(*s, generator=g, device="cuda") * 0.6).to(torch.bfloat16)
    q, k, v = mk(B, S, 128), mk(B, N, 128), mk(B, N, 128)
    lists = torch.randint(0, N, (B, C, Z), generator=g, device="cuda", dtype=torch.int32).sort(-1).values
    cnt = torch.randint(1, Z + 1, (B, C), generator=g, device="cuda", dtype=torch.int32)
    keep = torch.arange(Z, device="cuda")[None, None, :] < cnt[..., None]
    flat = lists[keep].contiguous()
    qh = torch.randint(0, C, (B, S), generator=g, device="cuda", dtype=torch.int32)
    qh[0, : S // 8] = 3                                            # a bucket of many items
    qh[1, : 60] = C - 1                                            # one of 60 queries: swept twice
    run = lambda: attention_hash_varlen(q, k, v, flat, cnt, qh, 128 ** -0.5, lse_dtype=torch.float32)
    outs = {}
    for which in ("wave-per-row", "wave"):
        ops.grouped_forward_kernel(which)
        try:
            outs[which] = run()
        finally:
            ops.grouped_forward_kernel(None)
    assert torch.equal(outs["wave-per-row"][0], outs["wave"][0]) and torch.equal(outs["wave-per-row"][1], outs["wave"][1])
    ops.force_generic_kernels(True)
    try:
        o2, l2 = run()
    finally:
        ops.force_generic_kernels(False)
    o1, l1 = outs["wave-per-row"]
    assert torch.allclose(o1.float(), o2.float(), atol=2e-2, rtol=1e-2)
    assert (l1 - l2).abs().max().item() < 1e-3
