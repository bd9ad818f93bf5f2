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
    extents take: fused for bf16 / fp16 at d = 128 with 65 536 keys or more, chunked otherwise)."""
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
