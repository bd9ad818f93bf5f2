"""The entry point that allocates nothing (fm_attention_hash_varlen_static) against the
workspace-taking fm_attention_hash_varlen, through the C ABI: same kernels, so the results must be
bit-identical, also on a second call with a smaller input that finds the static array holding the
first call's tables."""
import pytest
import torch

from fast_memory_amd import _lib, ops
from tests.util import dev, make_attn_case

pytestmark = pytest.mark.gpu


def _both(seed, B, S, N, C, Z, d, dtype):
    q, k, v, kh, cnt, qh = make_attn_case(seed, B, S, N, C, Z, d, dtype)
    q, k, v = dev(q, k, v)
    kh, cnt, qh = dev(kh.int(), cnt.int(), qh.int())
    scale = d ** -0.5
    ref_out, ref_lse = ops.attention_hash_varlen_i32(q, k, v, kh, cnt, qh, scale)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((B, S), float("nan"), dtype=torch.float32, device=q.device)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    ops.attention_hash_varlen_static_(q, k, v, kh, cnt, qh, scale, out, lse)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the wrapper allocated"
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       ref_out.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)), "out differs"
    assert torch.equal(lse.view(torch.int32), ref_lse.view(torch.int32)), "lse differs"


def test_static_scratch_entry_point_matches_workspace_entry_point():
    print("no-alloc: bf16 d=128 B=4 S=3000 N=20000 C=96 Z=512, then B=2 S=700 C=40", flush=True)
    _both(11, 4, 3000, 20000, 96, 512, 128, torch.bfloat16)      # ragged lists, staged MFMA kernel
    _both(12, 2, 700, 9000, 40, 256, 128, torch.bfloat16)        # smaller, over the first call's leftovers
    print("no-alloc: fp32 d=64 B=2 S=900 then S=100", flush=True)
    _both(13, 2, 900, 4096, 64, 128, 64, torch.float32)          # generic kernels
    _both(14, 1, 100, 2048, 16, 64, 64, torch.float32)


def test_static_scratch_entry_point_rejects_oversize():
    lib = _lib.load()
    H, C, Sq = 8, 4096, 1 << 20
    assert lib.fm_attention_hash_varlen_workspace(H, C, Sq) > _lib.FM_STATIC_SCRATCH_BYTES
    one = torch.zeros(1, device="cuda")
    p = one.data_ptr()          # never dereferenced: the size check comes before any launch
    rc = lib.fm_attention_hash_varlen_static(p, p, p, p, p, p, p, p, H, Sq, 1 << 20, 128, C, 1.0, 1, None)
    assert rc == 3 and b"static" in lib.fm_last_error()
