"""fp16 (FM_F16), the element type of the reference's own performance harness (triton_kernel.py:496): the
MFMA kernels of the forward path (projection, fused index build, query hash, staged gathered attention) and
the generic kernels of everything else, against the oracle on the same fp16 inputs."""
import math

import pytest
import torch

from oracle import fm_oracle as O
from tests.util import assert_attn_close, dev, gen, make_attn_case

pytestmark = pytest.mark.gpu
F16 = torch.float16


@pytest.fixture(scope="module")
def ops():
    from fast_memory_amd import ops as _ops
    from fast_memory_amd import _lib
    _lib.load()
    assert torch.cuda.is_available()
    return _ops


@pytest.mark.parametrize("H,C,N,d", [(2, 256, 1000, 128), (1, 130, 257, 64), (3, 7, 33, 24)])
def test_project_and_qhash_fp16(ops, H, C, N, d):
    g = gen(9100)
    A = torch.randn(H, C, d, generator=g).to(F16)
    K = torch.randn(H, N, d, generator=g).to(F16)
    Y = ops.project(*dev(A, K)).cpu()
    ref = O.project(A, K)
    assert torch.allclose(Y, ref, atol=2e-4 * math.sqrt(d), rtol=1e-5), (Y - ref).abs().max()
    h, sc = ops.qhash(*dev(A, K), return_scores=True)                 # the keys as queries
    assert torch.equal(h.cpu().long(), O.argmax_first(sc.cpu()))
    assert torch.allclose(sc.cpu(), O.qhash_scores(A, K), atol=2e-4 * math.sqrt(d), rtol=1e-5)
    if d == 128:                                                      # the streaming MFMA hash (no scores out)
        h2 = ops.qhash(*dev(A, K))
        assert torch.equal(h2, h)


def test_fused_build_fp16_bit_identical(ops):
    g = gen(9200)
    H, C, N, d, Z = 2, 70, 70001, 128, 512
    K = (torch.randn(H, N, d, generator=g) * 0.5).to(F16)
    A = torch.randn(H, C, d, generator=g).to(F16)
    Ad, Kd = dev(A, K)
    fused = ops.build_index(Ad, Kd, Z, fused=True)
    assert ops.last_build_info["path"] == "fused" and ops.last_build_info["rows_unresolved"] == 0
    assert torch.equal(fused, ops.build_index(Ad, Kd, Z, fused=False))
    assert torch.equal(fused.cpu().long(), O.argtopz(ops.project(Ad, Kd).cpu(), Z))


@pytest.mark.parametrize("B,S,N,C,Z,d", [(2, 300, 3000, 9, 500, 128),       # 33 queries per bucket: rows loaded straight into LDS
                                         (2, 600, 3000, 64, 200, 128),      # 9 per bucket, 128 items: staged, one item per workgroup
                                         (1, 2000, 2000, 8, 333, 128),      # 250 queries per bucket
                                         (2, 70, 300, 6, 40, 64)])          # generic kernel
def test_attention_forward_fp16(ops, B, S, N, C, Z, d):
    from fast_memory_amd import attention_hash_varlen
    q, k, v, kh, cnt, qh = make_attn_case(9300 + S, B, S, N, C, Z, d, F16, window="ref")
    if d == 128:
        name = ops.hash_attn_fwd_kernel_name(B, S, N, d, C, F16)
        assert name.startswith(("hash_attn_staged_kernel", "hash_attn_ring_kernel")) and "f16" in name, name
    out, lse = attention_hash_varlen(*dev(q, k, v, kh, cnt, qh), d ** -0.5)
    assert out.dtype == F16
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, d ** -0.5)
    assert_attn_close(out, lse, ro, rl, F16, "fp16 attention")
    # fp16 carries three more mantissa bits than bf16: the output is that much closer
    assert (out.float().cpu() - ro.float()).abs().max().item() < 4e-3


def test_attention_forward_fp16_many_queries_per_bucket(ops):
    # the kernels for buckets with many queries (two or three work items per workgroup; rows through staging registers,
    # or loaded straight into LDS), each forced, in fp16: against the oracle and bit for bit against each
    # other.  Buckets of 1, 64, 65, 128, 129 and 300 queries; ragged lists.
    from fast_memory_amd import attention_hash_varlen
    q, k, v, kh, cnt, qh = make_attn_case(9411, 2, 900, 4000, 10, 700, 128, F16, window="ref")
    sizes = [1, 64, 65, 128, 129, 300]
    pos = 0
    for b, n in enumerate(sizes):
        qh[0, pos:pos + n] = b
        pos += n
    qh[0, pos:] = 7
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 128 ** -0.5)
    outs = {}
    for which in ("staged-pairs", "ring", "ring-per-row", "staged-per-row", "wave", "wave-per-row"):
        ops.grouped_forward_kernel(which)
        try:
            out, lse = attention_hash_varlen(*dev(q, k, v, kh, cnt, qh), 128 ** -0.5)
        finally:
            ops.grouped_forward_kernel(None)
        assert_attn_close(out, lse, ro, rl, F16, f"fp16 {which}")
        outs[which] = (out, lse)
    assert torch.equal(outs["ring"][0], outs["staged-pairs"][0]) and torch.equal(outs["ring"][1], outs["staged-pairs"][1])
    for which in ("ring-per-row", "staged-per-row"):          # a launch per row: the same items, the same bits
        assert torch.equal(outs[which][0], outs["ring"][0]) and torch.equal(outs[which][1], outs["ring"][1])
    # (the kernel with a wave per item takes its softmax in steps of 16 keys, not 64: other roundings than the
    # rest, the same in both of its launch forms)
    assert torch.equal(outs["wave-per-row"][0], outs["wave"][0]) and torch.equal(outs["wave-per-row"][1], outs["wave"][1])


def test_composite_local_merge_and_backward_fp16(ops):
    from fast_memory_amd import Memory, attention_hash, fit_projection
    g = gen(9400)
    H, G, S, N, L, d, C, Z = 2, 2, 24, 70000, 24, 128, 16, 256
    keys = (torch.randn(H, N, d, generator=g) * 0.5).to(F16)
    vals = (torch.randn(H, N, d, generator=g) * 0.5).to(F16)
    q = (torch.randn(H, G * S, d, generator=g) * 0.5).to(F16)
    kl = (torch.randn(H, L, d, generator=g) * 0.5).to(F16)
    vl = (torch.randn(H, L, d, generator=g) * 0.5).to(F16)
    kd, vd, qd = dev(keys, vals, q)
    A = fit_projection(kd, C, iters=1)                                 # K-means through the fp16 hash kernel
    assert A.dtype == F16 and torch.allclose(A.float().norm(dim=-1), torch.ones(H, C, device="cuda"), atol=2e-3)
    out, lse = attention_hash(qd, kd, vd, A, Z, d ** -0.5)             # fused build + hash + attention
    lists = O.argtopz(ops.project(A, kd).cpu(), Z)
    qh, sc = ops.qhash(A, qd, return_scores=True)
    assert torch.equal(qh.cpu().long(), O.argmax_first(sc.cpu()))
    cnt = torch.full((H, C), Z)
    ro, rl = O.hashed_attention_gather(q, keys, vals, lists.reshape(-1), cnt, qh.cpu().long(), d ** -0.5)
    assert_attn_close(out, lse, ro, rl, F16, "attention_hash fp16")
    mem = Memory.build(kd, vd, A, Z)
    mo, ml = mem.attend_with_local(qd, *dev(kl, vl), d ** -0.5, n_groups=G, causal=True)
    lo, ll = O.local_attention(q.reshape(1, H * G, S, d), kl[None], vl[None], d ** -0.5, True)
    eo, el = O.lse_merge_closed_form(lo.reshape(H, G * S, d).float(), ll.reshape(H, G * S), ro.float(), rl)
    assert torch.allclose(mo.cpu().double(), eo.double(), atol=4e-3, rtol=1e-2)
    assert float((ml.cpu().double() - el.double()).abs().max()) < 2e-3
    # backward (the MFMA kernels; the partial rows of the form without atomics are bf16 for fp16 inputs too)
    dout = (torch.randn(H, G * S, d, generator=g) * 0.5).to(F16)
    dq, dk, dv = mem.attend_backward(dev(dout), qd, out, lse, d ** -0.5, q_hash=qh)
    rq, rk, rv = O.hashed_attention_backward_gather(q.float(), keys.float(), vals.float(), lists.reshape(-1), cnt,
                                                    qh.cpu().long(), out.float().cpu(), lse.cpu(), dout.float(),
                                                    d ** -0.5)
    for got, ref, name in ((dq, rq, "dq"), (dk, rk, "dk"), (dv, rv, "dv")):
        got = got.float().cpu().double()
        assert torch.allclose(got, ref, atol=3e-3 * max(1.0, ref.abs().max().item()), rtol=1e-2), \
            f"{name}: {(got - ref).abs().max().item():.3e}"
