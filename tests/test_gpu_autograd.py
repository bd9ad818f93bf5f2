"""The operators as autograd sees them: ``loss.backward()`` through the registered operators and through the
one-Function module forward, against fp64 autograd of a dense softmax over each query's keys."""
import os
import re
import subprocess
import sys

import pytest
import torch

from oracle import fm_oracle as O
from tests.util import assert_attn_close, dev, gen, make_attn_case

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _dense_reference(q, k, v, kh, cnt, qh, sm, w_out, w_lse):
    """fp64: per query a softmax over its bucket's keys, loss = sum(out * w_out) + sum(lse * w_lse) over the
    queries whose bucket is not empty; returns out, lse and the gradients w.r.t. q, k, v."""
    H, S, d = q.shape
    qd, kd, vd = (t.double().clone().requires_grad_(True) for t in (q, k, v))
    off = O.bucket_offsets(cnt)
    outs, lses = torch.zeros(H, S, d, dtype=torch.float64), torch.full((H, S), float("-inf"), dtype=torch.float64)
    loss = 0.0
    for h in range(H):
        for i in range(S):
            b = int(qh[h, i])
            c = int(cnt[h, b])
            if c == 0:
                continue
            idx = kh[int(off[h, b]):int(off[h, b]) + c].long()
            s = (kd[h, idx] @ qd[h, i]) * sm
            l = torch.logsumexp(s, 0)
            o = torch.softmax(s, 0) @ vd[h, idx]
            loss = loss + (o * w_out[h, i].double()).sum() + l * w_lse[h, i].double()
            outs[h, i], lses[h, i] = o.detach(), l.detach()
    loss.backward()
    return outs, lses, qd.grad, kd.grad, vd.grad


@pytest.mark.parametrize("dtype,B,S,N,C,Z,d", [(torch.float32, 2, 40, 300, 5, 48, 64),
                                               (torch.bfloat16, 2, 150, 900, 6, 200, 128)])
def test_registered_operator_backward_with_lse_gradient(dtype, B, S, N, C, Z, d):
    """torch.ops.fastmem.attention_hash_varlen: gradients flow to q, k and v through BOTH outputs (out and
    the log-sum-exp), as a caller needs that merges partial results with torch operations of its own."""
    from fast_memory_amd import attention_hash_varlen_op
    q, k, v, kh, cnt, qh = make_attn_case(8100 + S, B, S, N, C, Z, d, dtype, window="ref", std=0.7)
    g = gen(8101)
    w_out = (torch.randn(B, S, d, generator=g) * 0.5).to(dtype)
    w_lse = torch.randn(B, S, generator=g) * 0.5
    qd, kd, vd = (t.requires_grad_(True) for t in dev(q, k, v))
    out, lse = attention_hash_varlen_op(qd, kd, vd, *dev(kh, cnt, qh), d ** -0.5)
    assert out.requires_grad and lse.requires_grad and lse.dtype == torch.float32
    keep = (lse > -1e30).detach()
    loss = (out.float() * dev(w_out).float()).sum() + (torch.where(keep, lse, torch.zeros_like(lse)) * dev(w_lse)).sum()
    loss.backward()
    ro, rl, rq, rk, rv = _dense_reference(q, k, v, kh, cnt, qh, d ** -0.5, w_out, w_lse)
    assert_attn_close(out.detach(), lse.detach(), ro, torch.where(torch.isinf(rl), torch.full_like(rl, -3e38), rl),
                      dtype, "forward")
    for got, ref, name in ((qd.grad, rq, "dq"), (kd.grad, rk, "dk"), (vd.grad, rv, "dv")):
        got = got.float().cpu().double()
        tol = 1e-4 if dtype == torch.float32 else 2e-2 * max(1.0, ref.abs().max().item())
        assert torch.allclose(got, ref, atol=tol, rtol=1e-4 if dtype == torch.float32 else 2e-2), \
            f"{name}: max err {(got - ref).abs().max().item():.3e}"


def test_reference_operator_schema():
    """torch.ops.notbad.attention_hash_varlen takes exactly what the reference's host wrapper hands its
    operator (triton_kernel.py:75-106: queries sorted by bucket, one group per (row, bucket) pair, offsets)
    and returns what that wrapper expects (sorted order, base-2 LSE): the rest of the wrapper
    (triton_kernel.py:108-117), restated below, then yields the oracle's result."""
    import fast_memory_amd  # noqa: F401  (registers the operator)
    import math
    B, S, N, C, Z, d = 3, 70, 400, 7, 50, 64
    q, k, v, kh, cnt, qh = make_attn_case(8200, B, S, N, C, Z, d, torch.float32, window="ref")
    perm, gz, gc, go = O.group_queries(qh, C)                         # the reference's grouping (tk:75-84)
    q_sorted = torch.gather(q, 1, perm[..., None].expand(-1, -1, d)).contiguous()
    k_off = O.bucket_offsets(cnt)
    qs = dev(q_sorted).requires_grad_(True)
    o, lse2 = torch.ops.notbad.attention_hash_varlen(qs, *dev(k, v, kh, cnt, k_off, gz, gc, go), 0.2, S, N, d, C)
    # triton_kernel.py:108-117
    o_out = torch.empty_like(o)
    b_idx = torch.arange(B, device="cuda")
    o_out[b_idx[:, None], dev(perm)] = o.detach()
    lse = lse2.detach().to(q.dtype) * math.log(2)
    lse_out = torch.empty_like(lse)
    lse_out[b_idx[:, None], dev(perm)] = lse
    lse_out = torch.nan_to_num(lse_out, nan=0.0, posinf=torch.finfo(lse_out.dtype).max,
                               neginf=torch.finfo(lse_out.dtype).min)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 0.2)
    assert_attn_close(o_out, lse_out, ro, rl, torch.float32, "reference operator schema")
    # and it is differentiable where the reference's is not (triton_kernel.py:44-48)
    o.sum().backward()
    assert qs.grad is not None and bool(torch.isfinite(qs.grad).all()) and float(qs.grad.abs().sum()) > 0


@pytest.mark.parametrize("dtype,H,G,S,N,d,C,Z,topk", [
    (torch.float32, 2, 2, 24, 600, 64, 6, 40, 8),
    (torch.float32, 1, 3, 9, 70, 16, 3, 70, 5),            # every key in every list; three query heads per KV head
    (torch.float32, 2, 1, 33, 300, 128, 11, 7, 3),
    (torch.bfloat16, 2, 2, 20, 500, 128, 5, 60, 8),        # the MFMA kernels, forward and backward
    (torch.float16, 1, 4, 17, 400, 128, 7, 33, 6),
    (torch.bfloat16, 2, 2, 12, 300, 64, 4, 50, 8),         # head dimension 64: the backward on padded rows
])
def test_module_forward_backward_against_joint_softmax(dtype, H, G, S, N, d, C, Z, topk):
    """ring_cross_attention_approx (memory.py:421-425, one device): the output is the softmax over the
    union of each query's bucket and its causal local prefix, and loss.backward() gives the gradients of
    exactly that function w.r.t. q, k_self, v_self, k and v (fp64 autograd on the GPU's own lists and
    hashes)."""
    from fast_memory_amd import compute_centroids, ops, ring_cross_attention_approx
    g = gen(8300 + S)
    sm = d ** -0.5
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.6).to(dtype)
    q, kq, ks, vs, k, v = mk(1, H * G, S, d), mk(1, H * G, N, d), mk(1, H, S, d), mk(1, H, S, d), mk(1, H, N, d), mk(1, H, N, d)
    w = mk(1, H * G, S, d)
    cent0 = O.init_centroids(C, d, dtype)
    leaves = [t.requires_grad_(True) for t in dev(q, ks, vs, k, v)]
    qd, ksd, vsd, kd, vd = leaves
    out, hashes = ring_cross_attention_approx(qd, dev(kq), ksd, vsd, kd, vd, dev(cent0), sm, C, Z, centroid_topk=topk,
                                              return_hashes=True)
    (out * dev(w)).sum().backward()
    # the lists the forward built (same calls, deterministic)
    A = compute_centroids(dev(kq)[0], dev(cent0), C, G, topk, normalize=True).permute(1, 0, 2).contiguous()
    lists = ops.build_index(A, dev(k)[0].contiguous(), Z).cpu().long()                     # [H, C, Z]
    qh = hashes.cpu().long().reshape(H, G, S)
    q64, ks64, vs64, k64, v64 = (t.detach().cpu().double().requires_grad_(True) for t in leaves)
    ref = torch.zeros(1, H * G, S, d, dtype=torch.float64)
    rows = []
    for h in range(H):
        for gg in range(G):
            for t in range(S):
                idx = lists[h, qh[h, gg, t]]
                kk = torch.cat([k64[0, h, idx], ks64[0, h, :t + 1]])
                vv = torch.cat([v64[0, h, idx], vs64[0, h, :t + 1]])
                p = torch.softmax((kk @ q64[0, h * G + gg, t]) * sm, 0)
                rows.append(((h * G + gg, t), p @ vv))
    loss = 0.0
    for (hq, t), o in rows:
        ref[0, hq, t] = o.detach()
        loss = loss + (o * w[0, hq, t].double()).sum()
    loss.backward()
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert torch.allclose(out.detach().cpu().double(), ref, atol=tol, rtol=tol)
    for got, want, name in ((qd.grad, q64.grad, "dq"), (ksd.grad, ks64.grad, "dk_self"), (vsd.grad, vs64.grad, "dv_self"),
                            (kd.grad, k64.grad, "dk"), (vd.grad, v64.grad, "dv")):
        err = (got.cpu().double() - want).abs().max().item()
        bound = 2e-4 if dtype == torch.float32 else 2e-2 * max(1.0, want.abs().max().item())
        assert err <= bound, f"{name}: max err {err:.3e} (bound {bound:.1e})"


def test_module_backward_notices_a_memory_changed_in_place():
    """The keys and values of the memory reach the backward through save_for_backward (the reference keeps
    clones, memory.py:243-244): overwriting them in place between forward and backward -- a KV cache that
    moves on -- is an error autograd reports, not a gradient against the new contents."""
    from fast_memory_amd import ring_cross_attention_approx
    g = gen(8310)
    H, G, S, N, d, C, Z, topk = 2, 2, 16, 300, 64, 4, 32, 8
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.6).cuda()
    q, kq, ks, vs = mk(1, H * G, S, d).requires_grad_(True), mk(1, H * G, N, d), mk(1, H, S, d), mk(1, H, S, d)
    k_leaf, v = mk(1, H, N, d).requires_grad_(True), mk(1, H, N, d)
    k = k_leaf * 1.0                                    # a non-leaf that may be written in place
    out = ring_cross_attention_approx(q, kq, ks, vs, k, v, dev(O.init_centroids(C, d, torch.float32)), d ** -0.5, C, Z,
                                      centroid_topk=topk)
    k.mul_(2.0)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        out.sum().backward()


@pytest.mark.parametrize("S,L,chunk_entries", [(40, 56, None), (37, 61, None), (1, 9, None),   # one chunk; a last block of 5; decode
                                               (200, 200, 8 * 200), (203, 230, 8 * 230)])   # token chunks of 64
def test_local_attention_backward_bf16(S, L, chunk_entries, monkeypatch):
    from fast_memory_amd import autograd as fm_autograd, local_attention_backward, ops as _ops
    if chunk_entries:
        monkeypatch.setattr(fm_autograd, "_PREFIX_CHUNK_ENTRIES", chunk_entries)
    g = gen(8400)
    H, G, d = 2, 4, 128
    q = (torch.randn(H * G, S, d, generator=g) * 0.6).to(torch.bfloat16)
    k = (torch.randn(H, L, d, generator=g) * 0.6).to(torch.bfloat16)
    v = (torch.randn(H, L, d, generator=g) * 0.6).to(torch.bfloat16)
    w = (torch.randn(H * G, S, d, generator=g) * 0.5).to(torch.bfloat16)
    out, lse = _ops.local_attn_fwd(*dev(q, k, v), d ** -0.5, True)
    dq, dk, dv = local_attention_backward(dev(w), dev(q), dev(k), dev(v), out, lse, d ** -0.5, True)
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    s = torch.einsum("hgid,hjd->hgij", q64.view(H, G, S, d), k64) * d ** -0.5
    mask = torch.arange(L)[None, :] > torch.arange(S)[:, None] + (L - S)
    o = torch.einsum("hgij,hjd->hgid", torch.softmax(s.masked_fill(mask, float("-inf")), -1), v64)
    (o.reshape(H * G, S, d) * w.double()).sum().backward()
    for got, want, name in ((dq, q64.grad, "dq"), (dk, k64.grad, "dk"), (dv, v64.grad, "dv")):
        got = got.float().cpu().double()
        assert torch.allclose(got, want, atol=2e-2 * max(1.0, want.abs().max().item()), rtol=2e-2), \
            f"{name}: {(got - want).abs().max().item():.3e}"


def test_integration_snippet_runs_verbatim():
    """The ctypes binding that the integration guide prints for the reference's operator, executed as printed (in a process
    of its own: it registers the operator name this package registers too) and checked against the oracle."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    snippet = [b for b in blocks if "fm_attention_hash_varlen.argtypes" in b]
    assert len(snippet) == 1
    driver = '''
import sys, torch
sys.path.insert(0, %r)
from oracle import fm_oracle as O
from tests.util import make_attn_case, assert_attn_close
for dtype, d in ((torch.float32, 64), (torch.bfloat16, 128)):
    q, k, v, kh, cnt, qh = make_attn_case(8500, 2, 90, 500, 6, 64, d, dtype, window="ref")
    c = lambda t: t.cuda()
    out, lse = torch.ops.notbad.attention_hash_varlen(c(q), c(k), c(v), c(kh), c(cnt), c(qh), 0.17)
    ro, rl = O.hashed_attention_gather(q, k, v, kh, cnt, qh, 0.17)
    assert_attn_close(out, lse, ro, rl, dtype, "binding snippet of the integration guide")
print("snippet ok")
''' % ROOT
    r = subprocess.run([sys.executable, "-c", snippet[0] + driver], cwd=ROOT, capture_output=True, text=True,
                       timeout=110)
    assert r.returncode == 0 and "snippet ok" in r.stdout, r.stdout + r.stderr
