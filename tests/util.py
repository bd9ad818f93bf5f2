"""Shared helpers of the GPU parity tests: seeded CPU inputs, moved to the GPU
for the library and kept on the CPU for the oracle."""
import math

import torch

BF16_ATOL, BF16_RTOL = 2e-2, 1e-2      # attention output, bf16 inputs
F32_TOL = 1e-4                         # attention output, fp32 inputs
LSE_ATOL = 1e-3                        # fp32 natural-log LSE


def gen(seed):
    return torch.Generator().manual_seed(seed)


def dev(*ts):
    out = tuple(t.to("cuda") for t in ts)
    return out if len(out) > 1 else out[0]


def make_attn_case(seed, B, S, N, C, Z, d, dtype=torch.float32, window="ref", std=0.5):
    """Inputs in the style of the reference's own test (triton_kernel.py:300-322):
    q,k,v ~ N(0, std^2), uniformly random buckets and hashes, and a window mask
    that makes the lists ragged (and, for N > 32K, many buckets empty)."""
    g = gen(seed)
    q = (torch.randn(B, S, d, generator=g) * std).to(dtype)
    k = (torch.randn(B, N, d, generator=g) * std).to(dtype)
    v = (torch.randn(B, N, d, generator=g) * std).to(dtype)
    qh = torch.randint(0, C, (B, S), generator=g)
    kh = torch.stack([torch.stack([torch.randperm(N, generator=g)[:Z] for _ in range(C)]) for _ in range(B)])
    if window == "ref":
        if N > 32 * 1024:
            mask = torch.logical_and(24 * 1024 <= kh, kh < 24 * 1024 + 100)
        else:
            mask = kh < int(N * 0.9)
    else:
        mask = torch.ones_like(kh, dtype=torch.bool)
    return q, k, v, kh[mask], mask.sum(-1), qh


def assert_attn_close(out, lse, ref_out, ref_lse, dtype, what=""):
    out, lse = out.float().cpu(), lse.float().cpu()
    ref_out, ref_lse = ref_out.float(), ref_lse.float()
    empty = ref_lse < -1e30
    assert torch.equal(lse < -1e30, empty), f"{what}: empty-bucket rows differ"
    if dtype == torch.float32:
        assert torch.allclose(out, ref_out, atol=F32_TOL, rtol=F32_TOL), \
            f"{what}: out max err {(out - ref_out).abs().max().item():.3e}"
    else:
        assert torch.allclose(out, ref_out, atol=BF16_ATOL, rtol=BF16_RTOL), \
            f"{what}: out max err {(out - ref_out).abs().max().item():.3e}"
    err = (lse[~empty] - ref_lse[~empty]).abs().max().item() if (~empty).any() else 0.0
    assert err <= LSE_ATOL, f"{what}: lse max err {err:.3e}"
    assert (out[empty] == 0).all(), f"{what}: empty-bucket rows must be zero"
