"""CPU-side checks of the boundary: the library loads, exports every symbol the
header declares, and rejects bad arguments with status codes before touching
the GPU."""
import ctypes
import os
import re

import pytest

from fast_memory_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    syms = set()
    for name in ("fastmem.h", "fastmem_debug.h"):
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        syms |= set(re.findall(r"\b(fm_[a-z0-9_]+)\s*\(", text))
    return sorted(syms)


def test_production_header_declares_no_debug_hook():
    text = open(os.path.join(ROOT, "include", "fastmem.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    assert "fm_debug_" not in text


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    syms = header_symbols()
    assert len(syms) >= 20
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/fastmem.h but not exported"
        assert s in _lib.SIGNATURES, f"{s} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(syms)


def test_version_and_error_string():
    lib = _lib.load()
    assert lib.fm_version() >= 100
    assert isinstance(lib.fm_last_error(), bytes)


def test_argument_errors_are_status_codes():
    lib = _lib.load()
    assert lib.fm_argtopz_f32(None, 4, 0, 0, 1, None, None, None, 0, None) == 1  # N = 0
    assert b"fm_argtopz_f32" in lib.fm_last_error()
    assert lib.fm_project(None, None, None, 1, 1, 1, 1000, 1, 0, None) == 1      # d > FM_MAX_D
    assert lib.fm_qhash(None, None, None, None, 1, 1, 1, 8, 7, None) == 1        # bad dtype
    assert lib.fm_lse_merge(None, None, None, None, 5, 8, 0, None) == 1          # null pointers
    assert lib.fm_group_queries(None, 1, 1, 1, None, None, None, None, None, 0, None, 0, None) == 1
    # the entry points beyond the reference's operator validate the same way, before any device call
    assert lib.fm_index_append(None, None, 1, 1, None, None, None, None, 1, 1, 1, 1, 1, None, 0, None, None) == 1
    assert b"fm_index_append" in lib.fm_last_error()
    assert lib.fm_inverse_index(None, None, None, 1, 1, 1, 1, None, None, None, 0, None) == 1
    assert lib.fm_inverse_index_key_order(None, None, None, 1, 1, 1, 1, None, None, None, None, 0, None) == 1
    assert lib.fm_hash_attn_bwd(None, None, None, None, None, None, None, None, None, 1, None, None, None, None,
                                None, None, None, 1, 1, 1, 8, 1, 1.0, 0, None) != 0
    assert lib.fm_hash_attn_bwd_staged(*([None] * 18), 1, 1, 1, 64, 1, None, 1.0, 1, None, 0, None) != 0   # d = 64
    assert b"fm_hash_attn_bwd_staged" in lib.fm_last_error()
    assert lib.fm_segment_sum(None, None, None, None, None, 1, 1, 1, 8, 0, None) != 0
    assert lib.fm_lists_key_order(None, None, None, 3, 10, None, None, None) == 1   # null pointers
    assert b"fm_lists_key_order" in lib.fm_last_error()
    assert lib.fm_lists_key_order(None, None, None, 3, 0, None, None, None) == 1    # N = 0
    assert lib.fm_lists_key_order(None, None, None, 0, 10, None, None, None) == 0   # no list: nothing to do
    assert lib.fm_lists_key_order(4096, 4096, 4096, 1, 10, 4096, None, None) == 1    # in place: refused before any launch
    assert b"in place" in lib.fm_last_error()
    assert lib.fm_debug_mfma(None, 5120, 1, None, None) == 1                          # null pointers
    assert lib.fm_debug_mfma(4096, 100, 1, 4096, None) == 1                           # too few operands
    assert lib.fm_hash_attn_fwd_workspace(1000) >= 1000 * 4 and lib.fm_hash_attn_fwd_workspace(0) == 0
    p = 4096                                                                          # never dereferenced
    assert lib.fm_hash_attn_fwd_ws(p, p, p, p, p, p, p, p, p, 1000, p, p, 1, 64, 64, 128, 4, 1.0, 1, p, 16, None) == 3
    assert b"workspace" in lib.fm_last_error()                                        # a workspace that is too small
    # extents the launch shapes of the local attention cannot express are refused before any launch
    assert lib.fm_local_attn_fwd(p, p, p, p, p, 1, 1, 65535 * 128 + 1, 16, 128, 1.0, 1, 1, None) != 0
    assert b"fm_local_attn_fwd" in lib.fm_last_error()
    assert lib.fm_local_attn_fwd(p, p, p, p, p, 65536, 1, 16, 16, 128, 1.0, 1, 1, None) != 0
    with pytest.raises(ValueError):
        _lib.check(1)


def test_workspace_queries():
    lib = _lib.load()
    assert lib.fm_group_max_items(8, 2048, 32768) == 8 * (2048 + 512) + 1
    assert lib.fm_build_index_workspace(8, 2048, 1048576, 128, 16384, 1) == 1048576 * 4
    assert lib.fm_attention_hash_varlen_workspace(2, 16, 100) > 0
    assert lib.fm_group_queries_workspace(1, 8, 24) >= 8 * 4
    assert lib.fm_index_append_workspace(2, 3, 5) >= 2 * 3 * 8 * 4           # rows padded to 16 bytes
    assert lib.fm_hash_attn_bwd_staged_workspace(1000) >= 1000 * 512         # two bf16 rows of 128 per list entry
    assert lib.fm_inverse_index_workspace(1000, 1, 100) >= 3 * 1000 * 4
    assert lib.fm_inverse_index_workspace(0, 1, 100) == 0
    # two tables [H][C][N / 256 + 1] of words and the ranges' totals
    assert lib.fm_inverse_index_key_order_workspace(2, 10, 1000) >= 2 * 2 * 10 * 5 * 4 + 2 * 4 * 4
    assert lib.fm_inverse_index_key_order_workspace(0, 10, 1000) == 0


def test_ops_refuse_cpu_tensors():
    import torch
    from fast_memory_amd import ops
    with pytest.raises(RuntimeError):
        ops.project(torch.zeros(1, 2, 8), torch.zeros(1, 4, 8))


def test_local_attention_dispatch_rule():
    # host-only: which kernel fm_local_attn_fwd would launch (G, S, L, d, dtype; FM_F32 = 0, FM_BF16 = 1, FM_F16 = 2)
    lib = _lib.load()
    name = lambda *a: lib.fm_local_attn_fwd_kernel(*a).decode()
    assert name(8, 4096, 4096, 128, 1) == "local_attn_dense_kernel<bf16, 128>"
    assert name(8, 4096, 4096, 128, 2) == "local_attn_dense_kernel<f16, 128>"
    assert name(8, 4096, 4096, 64, 1) == "local_attn_dense_kernel<bf16, 64>"
    assert name(8, 4096, 4096, 256, 2) == "local_attn_dense_kernel<f16, 256>"
    assert name(8, 1, 4096, 128, 1) == "local_attn_decode_kernel"
    assert name(8, 1, 4096, 128, 2) == "local_attn_dense_kernel<f16, 128>"
    assert name(8, 4096, 4096, 96, 1) == "local_attn_generic_kernel"
    assert name(8, 4096, 4096, 128, 0) == "local_attn_generic_kernel"


def test_grouped_forward_dispatch_rule():
    # host-only: which kernel fm_hash_attn_fwd would launch (H, Sq, N, d, C, dtype)
    lib = _lib.load()
    name = lambda *a: lib.fm_hash_attn_fwd_kernel(*a).decode()
    assert name(8, 32768, 1048576, 128, 2048, 1) == "hash_attn_wave_kernel"           # 1 M keys, 16 queries / bucket
    assert name(8, 32768, 1048576, 128, 2048, 2) == "hash_attn_wave_kernel<f16>"
    assert name(8, 24 * 2048, 1048576, 128, 2048, 1) == "hash_attn_wave_kernel"       # ... 24
    assert name(8, 24 * 2048 + 1, 1048576, 128, 2048, 1) == "hash_attn_ring_kernel"   # ... more than 24
    assert name(1, 32768, 1048576, 128, 2048, 1) == "hash_attn_ring_kernel"           # ... a single row (one launch)
    assert name(8, 16384, 262144, 128, 1024, 1) == "hash_attn_ring_kernel"            # 256 K keys, 16 queries / bucket
    assert name(8, 8192, 262144, 128, 1024, 1) == "hash_attn_ring_kernel"             # ... 8 / bucket: too few buckets per row
    assert name(8, 16384, 1048576, 128, 4096, 1) == "hash_attn_wave_kernel"           # 4096 buckets, 4 queries / bucket
    assert name(8, 2047, 1048576, 128, 4096, 1) == "hash_attn_ring_kernel"            # ... too few queries per row
    assert name(8, 32768, (1 << 24) + 64, 128, 2048, 1) == "hash_attn_staged_kernel<1, 64-bit rows>"
    assert name(8, 8192, 32768, 128, 256, 1) == "hash_attn_ring_kernel"               # prefill chunk, 32 / bucket
    assert name(8, 131072, 65536, 128, 1024, 1) == "hash_attn_ring_kernel"       # reference harness, 128 / bucket
    assert name(1, 64, 262144, 128, 64, 1) == "hash_attn_mfma_kernel"                 # few, small work items
    assert name(1, 2048, 262144, 128, 64, 1) == "hash_attn_ring_kernel"               # few buckets, many queries each
    assert name(8, 8192, 1 << 25, 128, 256, 1) == "hash_attn_staged_kernel<1, 64-bit rows>"   # beyond 32-bit byte offsets
    assert name(8, 8192, 32768, 128, 256, 2) == "hash_attn_ring_kernel<f16>"          # fp16 (FM_F16 = 2)
    assert name(8, 4096, 32768, 128, 256, 2) == "hash_attn_ring_kernel<f16>"          # fp16, 16 / bucket
    assert name(1, 64, 1 << 25, 128, 64, 1) == "hash_attn_mfma_kernel"                # few small items, any N
    assert name(1, 512, 4096, 64, 64, 0) == "hash_attn_generic_kernel"                # fp32 / d != 128
    # launches per call: one per row where K and V of all rows are 512 MB or more and a row fills the device
    # twice over; one otherwise
    launches = lib.fm_hash_attn_fwd_launches
    assert launches(8, 32768, 1048576, 128, 2048, 1) == 8
    assert launches(8, 32768, 1048576, 128, 2048, 2) == 8
    assert launches(1, 32768, 1048576, 128, 2048, 1) == 1                             # a single row
    assert launches(8, 16384, 262144, 128, 1024, 1) == 8                              # 1 GB in all
    assert launches(8, 16384, 262144, 128, 512, 1) == 1                               # too few buckets per row
    assert launches(8, 16384, (1 << 24) + 64, 128, 1024, 1) == 1                      # ... for the staged kernel
    assert launches(8, 8192, 32768, 128, 256, 1) == 1                                 # 134 MB in all
    assert launches(64, 16384, 32768, 128, 1024, 1) == 1                              # 1 GB in all, rows of 16 MB
    assert launches(32, 16384, 65536, 128, 1024, 1) == 32                             # rows of 32 MB
    assert launches(8, 131072, 1048576, 128, 2048, 1) == 8                            # 64 queries / bucket
    assert launches(8, 32768, (1 << 24) + 64, 128, 2048, 1) == 8                      # staged kernel, 64-bit rows
    assert launches(8, 131072, 65536, 128, 1024, 2) == 1                              # reference harness
    assert launches(8, 32768, 1048576, 64, 2048, 0) == 1                              # generic kernels
    assert launches(1, 64, 1048576, 128, 64, 1) == 1                                  # few small items: gather kernel


def test_diagnostic_switches_need_the_environment_flag():
    """The process-wide switches of fastmem_debug.h take effect only where FASTMEM_DEBUG_HOOKS=1 was set before
    the library's first call; elsewhere the setters do nothing and the Python wrappers refuse.  Checked through
    a host-only query (which kernel fm_hash_attn_fwd would launch), in child processes with and without the flag."""
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from fast_memory_amd import _lib, ops\n"
            "lib = _lib.load()\n"
            "lib.fm_debug_force_generic(1)\n"
            "name = lib.fm_hash_attn_fwd_kernel(8, 8192, 32768, 128, 256, 1).decode()\n"
            "try:\n"
            "    ops.force_generic_kernels(True); refused = False\n"
            "except RuntimeError:\n"
            "    refused = True\n"
            "print(lib.fm_debug_hooks_enabled(), name, refused)\n") % ROOT
    for flag, want in ((None, "0 hash_attn_ring_kernel True"), ("0", "0 hash_attn_ring_kernel True"),
                       ("1", "1 hash_attn_generic_kernel False")):
        env = {k: v for k, v in os.environ.items() if k != "FASTMEM_DEBUG_HOOKS"}
        if flag is not None:
            env["FASTMEM_DEBUG_HOOKS"] = flag
        out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == want, (flag, out.stdout)
