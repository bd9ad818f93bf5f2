"""The query path under HIP graph capture: the hash of the queries and the entry point that allocates nothing
(fm_qhash -> fm_attention_hash_varlen_static, both through the C ABI) recorded once into a graph and replayed.
The library records kernels only (no memset or copy nodes), every replay is checked against an eager run on the
same inputs, with eager work and synchronisations between the replays, and the inputs change between replays
(a graph that had baked in results instead of work would show)."""
import pytest
import torch

from fast_memory_amd import _lib, ops
from tests.util import dev, gen, make_attn_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_hash_and_attention_replayed_from_a_graph(dtype):
    H, S, N, C, Z, d = 4, 1500, 6000, 48, 256, 128
    q, k, v, kh, cnt, _ = make_attn_case(41, H, S, N, C, Z, d, dtype)
    A = torch.randn(H, C, d, generator=gen(42)).to(dtype)
    q, k, v, A = dev(q, k, v, A)
    kh, cnt = dev(kh.int(), cnt.int())
    scale = d ** -0.5
    lib = _lib.load()
    dt = {torch.bfloat16: 1, torch.float16: 2}[dtype]

    def run(qh_buf, out_buf, lse_buf):
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.fm_qhash(A.data_ptr(), q.data_ptr(), qh_buf.data_ptr(), None, H, C, S, d, dt, st))
        _lib.check(lib.fm_attention_hash_varlen_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), kh.data_ptr(),
                                                       cnt.data_ptr(), qh_buf.data_ptr(), out_buf.data_ptr(),
                                                       lse_buf.data_ptr(), H, S, N, d, C, scale, dt, st))

    bufs = lambda: (torch.zeros(H, S, dtype=torch.int32, device="cuda"), torch.zeros_like(q),
                    torch.zeros(H, S, dtype=torch.float32, device="cuda"))
    qh_e, out_e, lse_e = bufs()
    qh_g, out_g, lse_g = bufs()
    run(qh_e, out_e, lse_e)          # the first call on a device also looks up the static array: not under capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(qh_g, out_g, lse_g)
    for rep in range(4):
        if rep:                       # new queries in place: the graph reads the same buffers
            q.copy_((torch.randn(H, S, d, generator=gen(50 + rep)) * 0.5).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        run(qh_e, out_e, lse_e)       # eager, between the replays, over the same static array
        torch.cuda.synchronize()
        assert torch.equal(qh_g, qh_e), f"replay {rep}: hashes differ"
        assert torch.equal(out_g.view(torch.int16), out_e.view(torch.int16)), f"replay {rep}: out differs"
        assert torch.equal(lse_g.view(torch.int32), lse_e.view(torch.int32)), f"replay {rep}: lse differs"
        assert float(out_g.float().abs().sum()) > 0
    ref_out, ref_lse = ops.attention_hash_varlen_i32(q, k, v, kh, cnt, qh_e, scale)
    assert torch.equal(out_g.view(torch.int16), ref_out.view(torch.int16)) and torch.equal(lse_g, ref_lse)


def test_build_hash_and_attention_in_one_graph():
    """Index build and query path recorded together: fm_qhash -> fm_build_index_fused -> fm_lists_key_order ->
    fm_attention_hash_varlen_static, all through the C ABI into one graph (kernels only: the build reads
    nothing back, its status word stays on the device and is looked at after the replays).  Keys, values and
    queries change between replays; every replay equals the eager run of the same calls bit for bit, and the
    lists equal those of the Python wrapper that does check the status."""
    dtype, dt = torch.bfloat16, 1
    H, S, N, C, Z, d = 2, 3000, 65536, 40, 512, 128
    g = gen(61)
    mk = lambda *shape: (torch.randn(*shape, generator=g) * 0.5).to(dtype).cuda()
    k, v, q, A = mk(H, N, d), mk(H, N, d), mk(H, S, d), mk(H, C, d)
    scale = d ** -0.5
    lib = _lib.load()
    ws_bytes = lib.fm_build_index_fused_workspace(H, C, N, d, Z, dt)
    assert ws_bytes > 0, "the shape must be one the fused build takes"
    cnt = torch.full((H, C), Z, dtype=torch.int32, device="cuda")
    off = (torch.arange(H * C, dtype=torch.int64, device="cuda") * Z)

    def bufs():
        return dict(ws=torch.empty(ws_bytes, dtype=torch.uint8, device="cuda"),
                    idx=torch.zeros(H, C, Z, dtype=torch.int32, device="cuda"),
                    idx_k=torch.zeros(H * C * Z, dtype=torch.int32, device="cuda"),
                    status=torch.zeros(_lib.FM_FUSED_STATUS_INTS, dtype=torch.int32, device="cuda"),
                    qh=torch.zeros(H, S, dtype=torch.int32, device="cuda"), out=torch.zeros_like(q),
                    lse=torch.zeros(H, S, dtype=torch.float32, device="cuda"))

    def run(b):
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.fm_qhash(A.data_ptr(), q.data_ptr(), b["qh"].data_ptr(), None, H, C, S, d, dt, st))
        _lib.check(lib.fm_build_index_fused(A.data_ptr(), k.data_ptr(), b["idx"].data_ptr(), None, H, C, N, d, Z, dt,
                                            b["ws"].data_ptr(), ws_bytes, b["status"].data_ptr(), st))
        _lib.check(lib.fm_lists_key_order(b["idx"].data_ptr(), off.data_ptr(), cnt.data_ptr(), H * C, N,
                                          b["idx_k"].data_ptr(), None, st))
        _lib.check(lib.fm_attention_hash_varlen_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), b["idx_k"].data_ptr(),
                                                       cnt.data_ptr(), b["qh"].data_ptr(), b["out"].data_ptr(),
                                                       b["lse"].data_ptr(), H, S, N, d, C, scale, dt, st))

    e, gb = bufs(), bufs()
    run(e)                               # first calls: kernel attributes, the static array's address
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(gb)
    for rep in range(3):
        if rep:
            k.copy_(mk(H, N, d))
            v.copy_(mk(H, N, d))
            q.copy_(mk(H, S, d))
        graph.replay()
        torch.cuda.synchronize()
        run(e)
        torch.cuda.synchronize()
        assert gb["status"].tolist()[1] == 0 and e["status"].tolist()[1] == 0
        for name in ("qh", "idx", "idx_k"):
            assert torch.equal(gb[name], e[name]), f"replay {rep}: {name} differs"
        assert torch.equal(gb["out"].view(torch.int16), e["out"].view(torch.int16)), f"replay {rep}: out differs"
        assert torch.equal(gb["lse"].view(torch.int32), e["lse"].view(torch.int32)), f"replay {rep}: lse differs"
    assert torch.equal(gb["idx"], ops.build_index(A, k, Z, fused=True))
    # the deferred check of the Python wrapper: same lists, nothing read back until asked
    idx2, st2 = ops.build_index(A, k, Z, fused=True, defer_check=True)
    assert st2.unresolved() == 0 and torch.equal(idx2, gb["idx"])


@pytest.mark.parametrize("eager_first", [True, False])
def test_paced_per_row_launches_replayed_from_a_graph(eager_first):
    """The kernel that gives every work item a wave of its own, in one launch per row (forced here on a small
    memory; dispatch takes it on large ones): each launch is followed by a one-thread kernel that sets the next
    launch's schedule from this one's duration, and both are recorded.  The schedules live in a table of the
    library whose address is asked for once per device -- not while a stream is being captured: captured
    first, the launches go unpaced.  Either way every replay gives the bits of the eager call."""
    H, S, N, C, Z, d = 5, 700, 9000, 64, 512, 128
    q, k, v, kh, cnt, qh = make_attn_case(77, H, S, N, C, Z, d, torch.bfloat16, window="all")   # full lists
    q, k, v = dev(q, k, v)
    kh, cnt, qh = dev(kh.int(), cnt.int(), qh.int())
    kh = kh.reshape(H, C, Z).sort(-1).values.reshape(-1).contiguous()      # ascending lists: what the pacing expects
    scale = d ** -0.5
    lib = _lib.load()

    def run(out_buf, lse_buf):
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.fm_attention_hash_varlen_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), kh.data_ptr(),
                                                       cnt.data_ptr(), qh.data_ptr(), out_buf.data_ptr(),
                                                       lse_buf.data_ptr(), H, S, N, d, C, scale, 1, st))

    bufs = lambda: (torch.zeros_like(q), torch.zeros(H, S, dtype=torch.float32, device="cuda"))
    out_e, lse_e = bufs()
    out_g, lse_g = bufs()
    ref_out, ref_lse = ops.attention_hash_varlen_i32(q, k, v, kh, cnt, qh, scale)   # (dispatch's kernel; also the
    torch.cuda.synchronize()                                                       # first use of the static array)
    ops.grouped_forward_kernel("wave-per-row")
    try:
        assert ops.hash_attn_fwd_kernel_name(H, S, N, d, C, torch.bfloat16) == "hash_attn_wave_kernel"
        if eager_first:
            run(out_e, lse_e)
            torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run(out_g, lse_g)
        for rep in range(5):
            if rep:
                q.copy_((torch.randn(H, S, d, generator=gen(90 + rep)) * 0.5).to(torch.bfloat16))
            graph.replay()
            torch.cuda.synchronize()
            run(out_e, lse_e)
            torch.cuda.synchronize()
            assert torch.equal(out_g.view(torch.int16), out_e.view(torch.int16)), f"replay {rep}: out differs"
            assert torch.equal(lse_g.view(torch.int32), lse_e.view(torch.int32)), f"replay {rep}: lse differs"
            assert float(out_g.float().abs().sum()) > 0
    finally:
        ops.grouped_forward_kernel(None)
    del ref_out, ref_lse
