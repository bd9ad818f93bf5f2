"""The synthetic-workload generators, pinned by moments: the mean cosine of a
vMF sample is the Bessel ratio A_p(kappa) = I_{p/2}(kappa) / I_{p/2-1}(kappa)."""
import math

import torch
from scipy.special import ive

from fast_memory_amd import synth


def bessel_ratio(p, kappa):
    return ive(p / 2.0, kappa) / ive(p / 2.0 - 1.0, kappa)


def test_vmf_mean_resultant_length():
    g = torch.Generator().manual_seed(5)
    for p, kappa in ((128, 20.0), (128, 30.0), (16, 5.0)):
        w = synth.vmf_w(40000, p, kappa, g, "cpu")
        assert abs(w.mean().item() - bessel_ratio(p, kappa)) < 4e-3, (p, kappa, w.mean().item())
        assert (w.abs() <= 1).all()


def test_vmf_samples_are_unit_and_centred():
    g = torch.Generator().manual_seed(6)
    mu = synth.unit_centres(3, 64, g, "cpu")
    x = synth.vmf_around(mu[torch.randint(0, 3, (6000,), generator=g)], 25.0, g)
    assert torch.allclose(x.norm(dim=-1), torch.ones(6000), atol=1e-5)
    assert (x @ mu.T).max(-1)[0].mean().item() > bessel_ratio(64, 25.0) - 0.02


def test_workloads_deterministic_and_shaped():
    cfg = synth.CONFIGS["c2"]
    a = synth.make_workload(cfg, "cpu", N=512, S=8, H=2)
    b = synth.make_workload(cfg, "cpu", N=512, S=8, H=2)
    assert torch.equal(a.keys, b.keys) and torch.equal(a.queries, b.queries)
    assert a.keys.shape == (2, 512, 128) and a.queries.shape == (2, 32, 128) and a.keys.dtype == torch.bfloat16
    c1 = synth.make_workload(synth.CONFIGS["c1"], "cpu")
    assert c1.keys.shape == (1, 4096, 64) and c1.queries.shape == (1, 512, 64) and c1.keys.dtype == torch.float32
    c5 = synth.make_workload(synth.CONFIGS["c5"], "cpu", N=1024, S=4, H=1)
    assert c5.k_local.shape == (1, 1024, 128)
    # query norm sqrt(d); key norms log-normal(0, 0.25)
    assert abs(a.queries.float().norm(dim=-1).mean().item() - math.sqrt(128)) < 0.2
    assert abs(a.keys.float().norm(dim=-1).log().std().item() - 0.25) < 0.03


def test_decode_lengths():
    L = synth.decode_lengths()
    assert len(L) == 64 and all(8192 <= n <= 131072 for n, _, _ in L)
    n, c, z = L[0]
    assert c == round(math.sqrt(n)) and z == round(4 * math.sqrt(n))
    assert L == synth.decode_lengths()
