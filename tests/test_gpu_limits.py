"""Shapes beyond what the fast kernels are sized for, which the reference takes without limit: lists longer
than FM_MAX_Z (memory.py:273 has no cap on n_results), memories of more than 2^24 keys, more than 16 query
heads per KV head in a decode batch."""
import pytest
import torch

from oracle import fm_oracle as O
from tests.util import BF16_ATOL, BF16_RTOL, LSE_ATOL, assert_attn_close, dev, gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from fast_memory_amd import ops as _ops
    from fast_memory_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return _ops


@pytest.mark.parametrize("rows,N,Z", [(3, 100000, 20000), (2, 70000, 40001), (1, 30000, 30000)])
def test_argtopz_longer_than_fm_max_z(ops, rows, N, Z):
    g = gen(9500 + Z)
    Y = torch.randn(rows, N, generator=g)
    Y[0, 1000:9000] = Y[0, 77]                                  # a run of 8000 equal values, partly inside the cut
    Y[-1, ::3] = 0.5
    got, vals = ops.argtopz(dev(Y), Z, return_values=True)
    ref = torch.sort(Y + 0.0, dim=-1, descending=True, stable=True)
    Zc = min(Z, N)
    assert got.shape == (rows, Zc)
    assert torch.equal(got.cpu().long(), ref.indices[:, :Zc]) and torch.equal(vals.cpu(), ref.values[:, :Zc])


def test_build_index_and_attention_with_long_lists(ops):
    from fast_memory_amd import Memory
    g = gen(9600)
    H, C, N, d, Z, S = 2, 3, 70000, 128, 20000, 40
    K = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    V = (torch.randn(H, N, d, generator=g) * 0.5).to(torch.bfloat16)
    A = torch.randn(H, C, d, generator=g).to(torch.bfloat16)
    q = (torch.randn(H, S, d, generator=g) * 0.5).to(torch.bfloat16)
    mem = Memory.build(*dev(K, V, A), Z)
    assert ops.last_build_info["path"] == "unfused"
    Y = ops.project(*dev(A, K)).cpu()
    assert torch.equal(mem.bucket_idx.cpu().long(), O.argtopz(Y, Z))
    out, lse = mem.attend(dev(q), d ** -0.5)
    qh = mem.hash(dev(q)).cpu().long()
    ro, rl = O.hashed_attention_gather(q, K, V, mem.bucket_idx.cpu().long().reshape(-1), torch.full((H, C), Z), qh,
                                       d ** -0.5)
    assert_attn_close(out, lse, ro, rl, torch.bfloat16, "Z = 20000")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_attention_over_more_than_2_24_keys(ops, dtype):
    """One row of 2^24 + 8192 keys (4.3 GB of K, as much of V): the staged kernel in its form with 64-bit row
    offsets, lists that name rows on both sides of the 4 GiB byte offset; against the oracle on the
    gathered rows and, for bf16, against the register-gather kernel."""
    N, d, C, Z, Sq = (1 << 24) + 8192, 128, 8, 512, 2048
    g = torch.Generator(device="cuda").manual_seed(9700)
    k = torch.empty(1, N, d, dtype=dtype, device="cuda").normal_(0, 0.5, generator=g)
    v = torch.empty(1, N, d, dtype=dtype, device="cuda").normal_(0, 0.5, generator=g)
    q = (torch.randn(1, Sq, d, generator=g, device="cuda") * 0.5).to(dtype)
    lists = torch.randint(0, N, (1, C, Z), generator=g, device="cuda", dtype=torch.int64)
    lists[0, :, ::2] = N - 1 - torch.randint(0, 8192, (C, Z // 2), generator=g, device="cuda")   # beyond 2^24
    lists[0, 0, 0], lists[0, 0, 1] = N - 1, 1 << 24
    qh = torch.randint(0, C, (1, Sq), generator=g, device="cuda", dtype=torch.int32)
    cnt = torch.full((1, C), Z, dtype=torch.int32, device="cuda")
    name = ops.hash_attn_fwd_kernel_name(1, Sq, N, d, C, dtype)
    assert "64-bit rows" in name, name
    flat = lists.to(torch.int32).reshape(-1).contiguous()
    out, lse = ops.attention_hash_varlen_i32(q, k, v, flat, cnt, qh, d ** -0.5)
    # oracle on the gathered rows
    rows = lists.reshape(-1)
    Ks, Vs = k[0, rows].cpu(), v[0, rows].cpu()
    ro, rl = O.hashed_attention_gather(q.cpu(), Ks[None], Vs[None], torch.arange(C * Z), cnt.cpu().long(),
                                       qh.cpu().long(), d ** -0.5)
    assert_attn_close(out, lse, ro, rl, dtype, "N > 2^24")
    ops.grouped_forward_kernel("staged-per-row")        # the same kernel as a launch per row (here: of the one row)
    try:
        op, lp = ops.attention_hash_varlen_i32(q, k, v, flat, cnt, qh, d ** -0.5)
    finally:
        ops.grouped_forward_kernel(None)
    assert torch.equal(op, out) and torch.equal(lp, lse)
    if dtype == torch.bfloat16:
        ops.grouped_forward_kernel("gather")
        try:
            og, lg = ops.attention_hash_varlen_i32(q, k, v, flat, cnt, qh, d ** -0.5)
        finally:
            ops.grouped_forward_kernel(None)
        assert torch.allclose(out.float(), og.float(), atol=BF16_ATOL, rtol=BF16_RTOL)
        assert float((lse - lg).abs().max()) <= LSE_ATOL


def test_decode_batch_with_32_query_heads_per_kv_head(ops):
    from fast_memory_amd import Memory, MemoryBatch
    g = torch.Generator(device="cuda").manual_seed(9800)
    H, G, d = 2, 32, 128
    mems = []
    for N, C, Z in ((3000, 12, 200), (5000, 20, 300)):
        K = torch.randn(H, N, d, generator=g, device="cuda").to(torch.bfloat16)
        V = torch.randn(H, N, d, generator=g, device="cuda").to(torch.bfloat16)
        A = torch.randn(H, C, d, generator=g, device="cuda").to(torch.bfloat16)
        mems.append(Memory.build(K, V, A, Z))
    q = torch.randn(len(mems), H, G, d, generator=g, device="cuda").to(torch.bfloat16)
    out, lse, h = MemoryBatch(mems).attend(q, d ** -0.5)
    assert out.shape == (2, H, G, d) and lse.shape == (2, H, G) and h.shape == (2, H, G)
    for s, m in enumerate(mems):
        hs = m.hash(q[s])
        assert torch.equal(hs, h[s])
        o1, l1 = m.attend(q[s], d ** -0.5, q_hash=hs)
        assert torch.allclose(out[s].float(), o1.float(), atol=BF16_ATOL, rtol=BF16_RTOL)
        assert float((lse[s] - l1).abs().max()) <= LSE_ATOL
