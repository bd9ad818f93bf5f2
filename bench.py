#!/usr/bin/env python3
"""Benchmark of the indexed-memory hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c5|c2|c1|c3|c4|tkperf]

One "step" is one pass of the query path over the whole synthetic batch, inputs
already resident in HBM: query hash -> grouping -> bucket-gathered attention ->
(dense local attention -> LSE merge, where the configuration has local keys).
``value`` is query-heads per second over K timed steps.  The index build
(projection + arg-top-Z) and the K-means that produces A are timed beside it
and reported in the same JSON line, as are the roofline figures of the
dominant kernel and a CPU baseline on a bounded sample of the same workload.
``--config tkperf`` is the shape of the reference's own performance harness
(triton_kernel.py:507-528), whose step is the whole composite ``attention_hash``:
index build + query hash + attention per call.
Prints exactly one JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

# the phase markers of the fused build and the forced kernels of the controls are diagnostic switches of the
# library, which take effect only in a process that asks for them before the library's first call
os.environ.setdefault("FASTMEM_DEBUG_HOOKS", "1")

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def ev_pair():
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def settle(fn, seconds=0.25):
    """Runs fn() for a quarter of a second before the warm-up steps.  The first process on a fresh machine has
    been seen to stall once, for some 40 ms, within its first launches of a kernel sequence; in a configuration
    whose step takes 0.1 ms that one stall, landing inside the timed steps, was most of their time."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        fn()
        torch.cuda.synchronize()


def timed(fn, reps=1, warm=1):
    """Average milliseconds of fn() over `reps` runs, HIP events on the current stream."""
    for _ in range(warm):
        fn()
    a, b = ev_pair()
    a.record()
    for _ in range(reps):
        r = fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps, r


def cpu_model():
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def cpu_threads():
    """Threads the CPU baseline uses: every core this process may use (the GPU boxes export their CPU share
    as OMP_NUM_THREADS, which can be fewer than the cores the host shows)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return n


def cpu_timed(fn, reps=3):
    """One untimed warm-up pass, then `reps` timed passes: (median seconds, all timed passes)."""
    fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], ts


def no_reuse_control(dev, reps=3, list_order="key", force=None):
    """fm_hash_attn_fwd on lists that name every key and value row exactly once: H = 8 rows of N = 2^24 keys,
    C = 2048 buckets (c5's number) of Z = 8192 keys = a seeded permutation of the keys, 16 queries per bucket
    (c5's average).  K and V are 69 GB, far beyond the 256 MB last-level cache, and no row is listed twice, so
    every gathered byte comes from HBM: the rate the gather kernel reaches here is an HBM rate, which the
    c5 figure (every key listed in ~32 buckets) is not.  Timed with the lists in the order the step reads
    them (``list_order``) and, beside it, in the other one.  ``force`` (a name :func:`ops.grouped_forward_kernel`
    takes) overrides the library's dispatch, which takes the kernel and the launch per row of c5 here too."""
    from fast_memory_amd import ops
    H, C, Z, d, per_bucket = 8, 2048, 8192, 128, 16
    N, Sq = C * Z, per_bucket * C
    k = torch.empty((H, N, d), dtype=torch.bfloat16, device=dev).normal_()
    v = torch.empty((H, N, d), dtype=torch.bfloat16, device=dev).normal_()
    g = torch.Generator(device=dev).manual_seed(4242)
    lists = torch.stack([torch.randperm(N, generator=g, device=dev).to(torch.int32) for _ in range(H)])
    q = torch.randn((H, Sq, d), generator=g, device=dev).to(torch.bfloat16)
    qh = (torch.arange(Sq, device=dev, dtype=torch.int32) % C).unsqueeze(0).expand(H, -1).contiguous()
    cnt = torch.full((H, C), Z, dtype=torch.int32, device=dev)
    off = ops.bucket_offsets(cnt)
    groups = ops.group_queries(qh, C)
    alg = H * C * Z * (2 * d * 2 + 4) + H * Sq * (2 * d * 2 + 4)
    ops.grouped_forward_kernel(force)
    res = {"kernel": ops.hash_attn_fwd_kernel_name(H, Sq, N, d, C, torch.bfloat16),
           "launches": ops.hash_attn_fwd_launches(H, Sq, N, d, C, torch.bfloat16),
           "workload": f"H={H}, N=2^24 keys/head (K+V {2 * H * N * d * 2 / 1e9:.1f} GB), C={C}, Z={Z}: lists = a "
                       f"seeded permutation, every row listed once; {per_bucket} queries per bucket",
           "algorithmic_bytes_per_launch": alg}
    flat = lists.reshape(-1)
    for order in ("value", "key"):          # as the permutation fell (what score order amounts to), then sorted
        if order == "key":
            flat = ops.lists_key_order(flat, off.reshape(-1), cnt.reshape(-1), N)
        run = lambda: ops.hash_attn_fwd(q, k, v, flat, off, cnt, groups, d ** -0.5)
        ms = min(timed(run, reps=1, warm=1 if i == 0 else 0)[0] for i in range(reps))
        out, lse = run()
        assert bool(torch.isfinite(lse).all())
        if order == list_order:
            res.update({"list_order": order, "launch_ms": ms, "gbs": alg / ms / 1e6,
                        "hbm_frac": alg / ms / 1e6 / HBM_PEAK_GBS})
        else:
            res["other_list_order"] = {"list_order": order, "launch_ms": ms, "gbs": alg / ms / 1e6}
    ops.grouped_forward_kernel(None)
    del k, v, lists, flat, q, out, lse
    torch.cuda.empty_cache()
    return res


def fused_phase_times(run):
    """Milliseconds of the phases of the fused index build, from HIP events the library records on
    its stream between them."""
    import ctypes
    from fast_memory_amd import _lib
    lib = _lib.load()
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(5)]
    for e in evs:
        e.record()                      # instantiates the underlying hipEvent_t
    torch.cuda.synchronize()
    arr = (ctypes.c_void_p * 5)(*[e.cuda_event for e in evs])
    lib.fm_debug_set_phase_events(arr, 5)
    try:
        run()
        torch.cuda.synchronize()
    finally:
        lib.fm_debug_set_phase_events(None, 0)
    names = ["thresholds_ms", "mfma_filter_ms", "select_ms", "repair_ms"]
    return {n: evs[i].elapsed_time(evs[i + 1]) for i, n in enumerate(names)}


def calibrate_copy(dev):
    """Launches copy_probe_kernel over 1 GiB: the kernel of known size that profiler HBM counters are
    scaled against."""
    from fast_memory_amd import _lib
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        _lib.check(_lib.load().fm_debug_copy(dst.data_ptr(), src.data_ptr(), src.numel(),
                                             torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()


def mfma_stream_probe(dev, iters=1000):
    """bf16 MFMA rate (TFLOP/s) of a register-resident loop of nothing but MFMAs on normally distributed
    operands: what the matrix pipes sustain on this device, for scale beside the published peak (the device
    is power-bound there and clocks the loop lower the more the operand bits toggle)."""
    from fast_memory_amd import _lib
    g = torch.Generator(device="cpu").manual_seed(11)
    operands = torch.randn(5120, generator=g).to(torch.bfloat16).to(dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    call = lambda: _lib.check(_lib.load().fm_debug_mfma(operands.data_ptr(), operands.numel(), iters, sink.data_ptr(),
                                                        torch.cuda.current_stream().cuda_stream))
    best_ms = min(timed(call, reps=1, warm=1)[0] for _ in range(5))
    return iters * 2.0 ** 33 / best_ms / 1e9


def hbm_traffic(kernel, workload, required=True):
    """Fabric-side bytes per launch of `kernel` on `workload`, measured offline with rocprofv3 --pmc (FETCH_SIZE,
    WRITE_SIZE) and kept as text under profiles/.  A kernel name the library's dispatch returns that has no entry
    there means the profile no longer describes what runs: that stops the benchmark (`required`)."""
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if os.path.exists(tpath):
        for ln in open(tpath):
            if ln.strip().startswith(f"{kernel}/{workload} ") and "=" in ln:
                return float(ln.split("=")[1])
    if required:
        sys.exit(f"bench.py: profiles/hbm_traffic.txt has no entry '{kernel}/{workload}': the dispatch launches a "
                 f"kernel whose traffic has not been profiled (run the rocprofv3 --pmc commands of profiles/ and add it)")
    return None


def fabric_gather_probe(dev, region_mib=64, passes=64):
    """GB/s of gather_probe_kernel: scattered 256-byte rows out of a region the last-level cache holds and an L2
    does not, every row once per sweep.  The rate the path last-level cache -> L2 sustains for the row fetches of
    the gathered attention; its L2 misses (HBM and that cache answer them together) cannot come faster."""
    from fast_memory_amd import _lib
    lib = _lib.load()
    src = torch.empty(region_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    call = lambda: _lib.check(lib.fm_debug_gather(src.data_ptr(), src.numel(), passes, sink.data_ptr(),
                                                  torch.cuda.current_stream().cuda_stream))
    best_ms = min(timed(call, reps=1, warm=1)[0] for _ in range(5))
    return max(src.numel(), 32 << 20) * passes / best_ms / 1e6


def distinct_rows_per_launch(lists, hit_mask, N):
    """Average over the rows (KV heads) of the number of distinct keys that the lists of a row's hit buckets
    name: what one launch over a row has to bring in from HBM at least once."""
    H = lists.shape[0]
    total = 0
    for h in range(H):
        seen = torch.zeros(N, dtype=torch.bool, device=lists.device)
        sel = lists[h][hit_mask[h]].reshape(-1).long()
        seen[sel.clamp_(0, N - 1)] = True
        total += int(seen.sum().item())
    return total / H


def index_build_record(cfg, wl, A, ws_bytes, dev, reps, km_ms=None, assign=None):
    """The index build of one configuration, timed and checked: keys/s of `reps` builds, its phases, the
    filter's MFMA rate, the selection's rate on a chunk of materialised Y, the time until the lists are ready
    for the attention (build + the key-ordered copy the step reads) and whether the lists are those of a stable
    descending sort of the GPU's own Y (sampled rows) and of the unfused build (every row)."""
    from fast_memory_amd import Memory, ops
    H, d, N, C, Z = cfg.H, cfg.d, cfg.N, cfg.C, cfg.Z
    e = 2 if cfg.dtype != torch.float32 else 4
    build = lambda: ops.build_index(A, wl.keys, Z, ws_bytes)
    # (three builds first: the first ones also pay for the allocator's first blocks of this size)
    build_ms, lists = timed(build, reps=reps, warm=3)
    rec = {"keys_per_s": H * N / (build_ms * 1e-3), "ms": build_ms, "keys": H * N, "timed_builds": reps,
           "path": dict(ops.last_build_info)}
    cnt = torch.full((H, C), lists.shape[2], dtype=torch.int32, device=dev)
    off = ops.bucket_offsets(cnt)
    ko_ms, _ = timed(lambda: ops.lists_key_order(lists.reshape(-1), off.reshape(-1), cnt.reshape(-1), N), reps=3, warm=1)
    rec["lists_key_order_ms"] = ko_ms
    rec["ready_for_attention_ms"] = build_ms + ko_ms
    rec["ready_for_attention_keys_per_s"] = H * N / ((build_ms + ko_ms) * 1e-3)
    if rec["path"].get("path") == "fused":
        ph = fused_phase_times(build)
        gemm_flops = 2.0 * H * C * N * d
        ph["filter_tflops"] = gemm_flops / ph["mfma_filter_ms"] / 1e9
        ph["filter_mfma_frac"] = ph["filter_tflops"] / BF16_MFMA_PEAK_TFLOPS
        ph["mfma_stream_probe_tflops"] = mfma_stream_probe(dev)
        ph["filter_vs_mfma_stream_probe"] = ph["filter_tflops"] / ph["mfma_stream_probe_tflops"]
        rec["fused_phases_ms"] = ph
        kern = ops.fused_filter_kernel_name(H, C, N, d, Z, cfg.dtype)
        rec["filter_roofline"] = {"kernel": kern, "bound": "mfma", "achieved": ph["filter_tflops"],
                                  "peak": BF16_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": ph["filter_mfma_frac"],
                                  "traffic": hbm_traffic(kern, cfg.name), "algorithmic_flops_per_launch": gemm_flops,
                                  "avg_launch_ms": ph["mfma_filter_ms"],
                                  "vs_mfma_stream_probe": ph["filter_vs_mfma_stream_probe"]}
    # component kernels of the unfused build on one chunk of rows: projection (a fill of Y) and arg-top-Z
    # (a read of Y): the selection's GB/s is quoted on the latter
    rows = min(C, max(1, min(2048, ws_bytes // (N * 4))))
    Asub = A[:1, :rows].contiguous()
    proj_ms, Y = timed(lambda: ops.project(Asub, wl.keys[:1]), reps=3, warm=1)
    sel_ms, sel_lists = timed(lambda: ops.argtopz(Y, Z), reps=3, warm=1)
    proj_flops = 2.0 * rows * N * d
    proj_bytes = rows * N * 4 + (rows + N) * d * e
    sel_bytes = rows * N * 4 + rows * min(Z, N) * 4
    rec["unfused_parts"] = {
        "chunk_rows": rows,
        "project": {"ms": proj_ms, "tflops": proj_flops / proj_ms / 1e9,
                    "mfma_frac": proj_flops / proj_ms / 1e9 / BF16_MFMA_PEAK_TFLOPS,
                    "hbm_gbs": proj_bytes / proj_ms / 1e6, "hbm_frac": proj_bytes / proj_ms / 1e6 / HBM_PEAK_GBS},
        "argtopz": {"ms": sel_ms, "hbm_gbs": sel_bytes / sel_ms / 1e6,
                    "hbm_frac": sel_bytes / sel_ms / 1e6 / HBM_PEAK_GBS}}
    rec["select_gbs"] = sel_bytes / sel_ms / 1e6
    rec["select_hbm_frac"] = rec["select_gbs"] / HBM_PEAK_GBS
    # the lists against the definition (stable descending sort of the GPU's own fp32 Y, first Z) on the rows of
    # that chunk spread 64 apart, and against the unfused build on every row
    pick = torch.arange(0, rows, max(1, rows // 64), device=dev)
    ref = torch.sort(Y[0, pick] + 0.0, dim=-1, descending=True, stable=True).indices[:, :min(Z, N)]
    same_def = bool(torch.equal(ref, lists[0, pick].long())) and bool(torch.equal(ref, sel_lists[0, pick].long()))
    del Y, ref, sel_lists
    same_unfused = None
    if rec["path"].get("path") == "fused":
        unfused = ops.build_index(A, wl.keys, Z, ws_bytes, fused=False)
        same_unfused = bool(torch.equal(unfused, lists))
        del unfused
    rec["lists_bit_exact"] = {"sampled_rows_vs_stable_sort_of_gpu_Y": same_def, "rows_sampled": int(pick.numel()),
                              "every_row_vs_unfused_build": same_unfused}
    if km_ms is not None:
        rec.update({"kmeans_ms": km_ms, "kmeans_iters": cfg.kmeans_iters, "kmeans_assign": assign})
    return rec, lists


def kmeans_record(cfg, wl, dev):
    """A by spherical K-means on the keys (timed), and its assignment step alone."""
    from fast_memory_amd import fit_projection, ops
    H, d, N, C = cfg.H, cfg.d, cfg.N, cfg.C
    km_ms, A = timed(lambda: fit_projection(wl.keys, C, iters=cfg.kmeans_iters), reps=2, warm=2)
    assign = None
    if cfg.dtype != torch.float32 and d == 128:
        assign_ms, _ = timed(lambda: ops.qhash(A, wl.keys), reps=3, warm=1)
        assign_tflops = 2.0 * H * C * N * d / assign_ms / 1e9
        assign = {"ms": assign_ms, "tflops": assign_tflops, "mfma_frac": assign_tflops / BF16_MFMA_PEAK_TFLOPS}
    return km_ms, A, assign


def bench_decode_batch(args):
    """Config 3: decode batch of 64 sequences with memories of 8192..131072 keys, 8 KV heads x 4 query
    heads, one token each, merged with dense attention over 512 local keys per sequence."""
    from fast_memory_amd import Memory, MemoryBatch, fit_projection, ops, synth
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    base = synth.CONFIGS["c2"]
    H, G, d = base.H, base.G, base.d
    lens = synth.decode_lengths()
    sm_scale = d ** -0.5
    t0 = time.time()
    mems, qs, kls, vls = [], [], [], []
    build_ms = 0.0
    for s, (N, C, Z) in enumerate(lens):
        cfg = synth.Config(f"c3-seq{s}", base.dtype, H, G, d, N, C, Z, 1, 256, 20.0, 2, 512, 1003 + s)
        wl = synth.make_workload(cfg, dev)
        A = fit_projection(wl.keys, C, iters=2)
        ms, mem = timed(lambda: Memory.build(wl.keys, wl.values, A, Z), reps=1, warm=0)
        build_ms += ms
        mems.append(mem)
        qs.append(wl.queries.reshape(H, G, d))
        kls.append(wl.k_local)
        vls.append(wl.v_local)
    batch = MemoryBatch(mems)
    q = torch.stack(qs)
    kl, vl = torch.stack(kls), torch.stack(vls)
    n_seq = len(lens)
    total_keys = sum(n for n, _, _ in lens) * H
    torch.cuda.synchronize()
    log(f"[bench] c3: {n_seq} memories built in {time.time() - t0:.1f}s wall, index builds {build_ms:.1f} ms "
        f"for {total_keys} keys")
    evs = []

    def step(record=True, events=True):
        if events:
            a, b = ev_pair()
            a.record()
        mo, ml, h = batch.attend(q, sm_scale)
        if events:
            b.record()
        L = kl.shape[2]
        lo, ll = ops.local_attn_fwd(q.reshape(n_seq * H * G, 1, d), kl.reshape(n_seq * H, L, d),
                                    vl.reshape(n_seq * H, L, d), sm_scale, True)
        from fast_memory_amd import update_out_and_lse
        out, lse = update_out_and_lse(None, None, lo.reshape(n_seq, H, G, d), ll.reshape(n_seq, H, G))
        out, lse = update_out_and_lse(out.contiguous(), lse.contiguous(), mo, ml)
        if record:
            evs.append((a, b))
        return out, lse, h

    settle(lambda: step(False))
    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, lse, h = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    qheads = n_seq * H * G
    attn_ms = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
    # the same step recorded once into a HIP graph and replayed (the library records kernels only; torch's
    # allocator serves the step's tensors from the graph's own pool): what a serving loop that replays pays
    graph_replay = None
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g_out, g_lse, g_h = step(False, events=False)
        for _ in range(max(args.warmup, 2)):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        g_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        graph_replay = {"ms_per_step": g_ms, "value": qheads / (g_ms * 1e-3),
                        "same_bits_as_eager": bool(torch.equal(g_out, out) and torch.equal(g_lse, lse) and torch.equal(g_h, h))}
        log(f"[bench] c3 step replayed from a HIP graph: {g_ms:.3f} ms {graph_replay}")
    except Exception as exc:  # a graph that cannot be captured here is reported, not fatal
        log(f"[bench] HIP graph capture of the c3 step failed: {exc!r}")
    hc = h.cpu()
    alg_bytes = 0
    for s, (N, C, Z) in enumerate(lens):
        for hh in range(H):
            alg_bytes += len(set(hc[s, hh].tolist())) * Z * (2 * d * 2 + 4) + C * d * 2
    alg_bytes += qheads * (2 * d * 2 + 4)
    achieved = alg_bytes / attn_ms / 1e6
    # CPU baseline: whole sequences (all heads, hash + bucket attention + local attention + merge), one
    # after the other until the time budget is used
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import cpu_path
        threads = cpu_threads()
        torch.set_num_threads(threads)

        def seq_pass(s_i):
            m = mems[s_i]
            Kc, Vc, Ac, Lc = m.keys.cpu(), m.values.cpu(), m.A.cpu(), m.bucket_idx.cpu().long()
            qc, klc, vlc = q[s_i].cpu(), kl[s_i].cpu(), vl[s_i].cpu()
            return sum(cpu_path.time_query_path(qc[hh], Kc[hh], Vc[hh], Ac[hh], Lc[hh], sm_scale, klc[hh], vlc[hh])
                       for hh in range(H))

        # pilot (also the warm-up): sequences one after the other until a quarter of the budget is used; the
        # same sequences are then timed three times and the median pass is reported
        t_pilot, seqs = 0.0, 0
        while seqs < n_seq and t_pilot < args.cpu_seconds / 4.0:
            t_pilot += seq_pass(seqs)
            seqs += 1
        passes = sorted(sum(seq_pass(s_i) for s_i in range(seqs)) for _ in range(3))
        n_done, t_total = seqs * H * G, passes[1]
        cpu = {"value": n_done / t_total, "unit": "query-heads/s", "cores": threads, "kind": "port",
               "cpu_model": cpu_model(), "host_cpu_count": os.cpu_count(),
               "protocol": "1 warm-up pass + 3 timed passes, median", "pass_seconds": passes,
               "sample": f"sequences 0..{seqs - 1} of {n_seq} (all {H} KV heads, {G} query heads each): hash + "
                         f"per-bucket gathered softmax attention + local attention over 512 keys + merge"}
        log(f"[bench] CPU port ({threads} threads): {cpu['value']:.0f} query-heads/s on {seqs} sequences")
    line = {
        "metric": "hashed-attn query-heads/s", "value": qheads / (ms_per_step * 1e-3), "unit": "query-heads/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"c3-varlen-decode-bf16: {n_seq} sequences, memory lengths {min(l[0] for l in lens)}.."
                               f"{max(l[0] for l in lens)} keys, H={H}, G={G}, d={d}, C=round(sqrt N), "
                               f"Z=round(4 sqrt N), 1 token per query head ({qheads} query-heads), 512 local keys",
                   "step": "batched hash + gather attention (one launch) + local attention + merge"},
        "roofline": {"kernel": "decode_hash_attn_kernel", "bound": "hbm", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": hbm_traffic("decode_hash_attn_kernel", "c3-varlen-decode-bf16"),
                     "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_ms": attn_ms},
        "cpu_baseline": cpu,
        "index_build": {"keys_per_s": total_keys / (build_ms * 1e-3), "ms": build_ms, "keys": total_keys},
        "graph_replay": graph_replay,
    }
    log(f"[bench] c3 step {ms_per_step:.3f} ms -> {line['value'] / 1e6:.2f} M query-heads/s; decode kernel "
        f"{attn_ms:.3f} ms = {achieved:.0f} GB/s algorithmic")
    print(json.dumps(line), flush=True)


def bench_reference_harness(args):
    """The reference's own performance harness (triton_kernel.py:404-412, 475-489, 507-528): 8 rows x 4
    groups x 32768 queries, 65536 keys, d = 128, 1024 buckets of 3072 keys, q / k / v / centroids ~ N(0,1);
    one step = attention_hash(q, k, v, centroids, bucket_size, sm_scale), i.e. index build + query hash +
    grouping + attention, and the figure it prints is the dense-equivalent 4*B*G*S*N*d flops per second.
    fp16 as in the reference (triton_kernel.py:496); ``--tk-dtype bf16`` runs the same shape in bf16."""
    from fast_memory_amd import attention_hash, ops
    B, G, S, N, d, C, Z = 8, 4, 32768, 65536, 128, 1024, 3072
    Sq = G * S
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator(device="cpu").manual_seed(1006)
    tk_dtype = torch.float16 if args.tk_dtype == "fp16" else torch.bfloat16
    mk = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float32).to(tk_dtype).to(dev)
    k, v, centroids = mk(B, N, d), mk(B, N, d), mk(B, C, d)
    q = torch.cat([mk(1, Sq, d) for _ in range(B)])
    sm_scale = d ** -0.5
    ws_bytes = int(args.workspace_gib * (1 << 30))

    # the parts, each on its own
    build_ms, lists = timed(lambda: ops.build_index(centroids, k, Z, ws_bytes), reps=3, warm=3)
    hash_ms, qh = timed(lambda: ops.qhash(centroids, q), reps=3, warm=1)
    group_ms, groups = timed(lambda: ops.group_queries(qh, C), reps=3, warm=1)
    off = ops.bucket_offsets(torch.full((B, C), Z, dtype=torch.int32, device=dev))
    cnt = torch.full((B, C), Z, dtype=torch.int32, device=dev)
    # attention_hash reorders the lists by key below 96 queries per bucket; this shape has 128 and reads them as built
    from fast_memory_amd.hash_attention import sorts_lists
    ko_ms, flat = None, lists.reshape(-1)
    if sorts_lists(Sq, C):
        ko_ms, flat = timed(lambda: ops.lists_key_order(lists.reshape(-1), off.reshape(-1), cnt.reshape(-1), N),
                            reps=3, warm=1)
    attn_ms, (mo, ml) = timed(lambda: ops.hash_attn_fwd(q, k, v, flat, off, cnt, groups, sm_scale), reps=5, warm=2)

    step = lambda: attention_hash(q, k, v, centroids, Z, sm_scale)
    settle(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out, lse = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    qheads = B * Sq
    value = qheads / (ms_per_step * 1e-3)
    dense_equiv_tflops = 4.0 * B * Sq * N * d / ms_per_step / 1e9          # what the reference prints
    hit = int((groups.bin_count > 0).sum().item())
    alg_bytes = hit * Z * (2 * d * 2 + 4) + qheads * (2 * d * 2 + 4)
    alg_flops = 4.0 * d * Z * qheads
    achieved = alg_bytes / attn_ms / 1e6
    attn_kernel = ops.hash_attn_fwd_kernel_name(B, Sq, N, d, C, tk_dtype)
    roofline = {"kernel": attn_kernel, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": hbm_traffic(attn_kernel, "tkperf"),
                "algorithmic_bytes_per_launch": alg_bytes, "avg_launch_ms": attn_ms, "hit_buckets": hit,
                "mfma_tflops": alg_flops / attn_ms / 1e9,
                "mfma_frac": alg_flops / attn_ms / 1e9 / BF16_MFMA_PEAK_TFLOPS,
                "note": "128 queries per bucket on average: 127 flop per algorithmic byte; the rows come from the "
                        "last-level cache, not from HBM; the kernel is bound by the MFMA and softmax work of a SIMD, "
                        "which issue one after the other, and by the wait for the next tile's rows"}
    log(f"[bench] tkperf step {ms_per_step:.2f} ms = {dense_equiv_tflops:.0f} dense-equivalent TFLOP/s; build "
        f"{build_ms:.2f}, hash {hash_ms:.2f}, group {group_ms:.2f}, attention {attn_ms:.2f} ms "
        f"({achieved:.0f} GB/s algorithmic, {roofline['mfma_tflops']:.0f} TFLOP/s)"
        + (f"; lists in key order {ko_ms:.2f} ms" if ko_ms is not None else ""))

    if args.calibrate_copy:
        calibrate_copy(dev)

    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        from oracle import cpu_path
        threads = cpu_threads()
        torch.set_num_threads(threads)
        K0, V0, A0 = k[0].cpu(), v[0].cpu(), centroids[0].cpu()
        r = 32
        tb0 = time.perf_counter()
        cpu_lists = cpu_path.build_rows(A0[:r], K0, Z)
        t_build = time.perf_counter() - tb0
        Yg = ops.project(centroids[:1, :r].contiguous(), k[:1])[0].cpu()
        ref_lists = torch.sort(Yg + 0.0, dim=-1, descending=True, stable=True)[1][:, :Z]
        lists0 = lists[0].cpu().long()
        # the query path of rows 0.. until the time budget is used (the cost is per bucket gathered)
        n_total, t_total, rows_used = 0, 0.0, 0
        while rows_used < B and t_total < args.cpu_seconds:
            b = rows_used
            t_total += cpu_path.time_query_path(q[b].cpu(), k[b].cpu(), v[b].cpu(), centroids[b].cpu(),
                                                lists[b].cpu().long(), sm_scale)
            n_total += Sq
            rows_used += 1
        t_row = t_total / rows_used + C * t_build / r                     # one row: its build + its queries
        cpu = {"value": Sq / t_row, "unit": "query-heads/s", "cores": threads, "kind": "port",
               "cpu_model": cpu_model(), "host_cpu_count": os.cpu_count(), "protocol": "one pass (rows in sequence)",
               "sample": f"rows 0..{rows_used - 1} of {B}: hash + per-bucket gathered softmax attention of all {Sq} "
                         f"queries of each ({t_total:.2f} s), plus the index build of {r} of {C} bucket rows of row 0 "
                         f"({t_build:.2f} s) extrapolated to the {C}"}
        sel = torch.linspace(0, Sq - 1, 4096).long()
        co, cl, ch = cpu_path.hashed_attention(q[0].cpu()[sel], K0, V0, A0, lists0, sm_scale)
        same = qh[0].cpu().long()[sel] == ch
        parity = {"hash_agree_frac": same.float().mean().item(),
                  "out_max_abs_err": (out[0].float().cpu()[sel][same] - co[same]).abs().max().item(),
                  "lse_max_abs_err": (lse[0].float().cpu()[sel][same] - cl[same]).abs().max().item(),
                  "bucket_rows_bit_exact_vs_cpu_stable_sort_of_gpu_Y": bool(torch.equal(ref_lists, lists0[:r]))}
        log(f"[bench] cpu baseline: {cpu['value']:.1f} query-heads/s on {threads} threads; parity {parity}")

    line = {
        "metric": "hashed-attn query-heads/s", "value": value, "unit": "query-heads/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16" if tk_dtype == torch.float16 else "bf16",
        "data": "synthetic",
        "config": {"workload": f"tkperf: the reference's performance harness, {B} rows x {G} groups x {S} queries, "
                               f"N={N} keys, d={d}, C={C}, Z={Z}, q/k/v/centroids ~ N(0,1)",
                   "step": "attention_hash: index build + query hash + grouping + gather attention"},
        "roofline": roofline, "cpu_baseline": cpu,
        "dense_equivalent_tflops": dense_equiv_tflops,
        "step_parts_ms": {"index_build": build_ms, "lists_key_order": ko_ms, "qhash": hash_ms, "group": group_ms,
                          "attention": attn_ms},
        "index_build": {"keys_per_s": B * N / (build_ms * 1e-3), "ms": build_ms, "keys": B * N,
                        "path": dict(ops.last_build_info)},
        "parity_spot_check": parity,
    }
    print(json.dumps(line), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c5", choices=["c1", "c2", "c3", "c4", "c5", "tkperf"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-backward", action="store_true", help="skip timing the backward of the gathered attention")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--workspace-gib", type=float, default=8.0)
    ap.add_argument("--tk-dtype", default="fp16", choices=["fp16", "bf16"],
                    help="element type of --config tkperf (the reference's harness runs fp16)")
    ap.add_argument("--list-order", default="key", choices=["key", "value"],
                    help="order of a bucket's list as the gathered attention reads it: ascending key index (the "
                         "copy Memory keeps for its attention) or descending score as torch.topk leaves it")
    ap.add_argument("--head-dim", type=int, default=0, choices=[0, 64, 128, 256],
                    help="run the configuration's shape with another head dimension (the reference kernel is "
                         "generic in d_head); 0 keeps the configuration's own")
    ap.add_argument("--no-c4-build", action="store_true",
                    help="with --config c5: leave out the index build of c4 (the configuration the keys/s half of "
                         "the metric is quoted on), which otherwise runs after the c5 step and goes into the same line")
    ap.add_argument("--no-control", action="store_true",
                    help="skip the no-reuse control of the attention roofline (69 GB of K and V listed once)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch copy_probe_kernel over 1 GiB (the known-size kernel profiler "
                         "HBM counters are scaled against)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures one GPU (one MI355X holds a whole memory at its real "
                 "shape); run it with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; there is no CPU path to time")

    from fast_memory_amd import Memory, fit_projection, ops, synth, update_out_and_lse
    from fast_memory_amd import _lib
    _lib.load()
    if args.config == "c3":
        return bench_decode_batch(args)
    if args.config == "tkperf":
        return bench_reference_harness(args)
    cfg = synth.CONFIGS[args.config]
    if args.head_dim and args.head_dim != cfg.d:
        import dataclasses
        cfg = dataclasses.replace(cfg, d=args.head_dim, name=f"{cfg.name}-d{args.head_dim}")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    H, G, d, N, C, Z, S = cfg.H, cfg.G, cfg.d, cfg.N, cfg.C, cfg.Z, cfg.S
    Sq = G * S
    e = 2 if cfg.dtype == torch.bfloat16 else 4
    sm_scale = d ** -0.5
    ws_bytes = int(args.workspace_gib * (1 << 30))

    t0 = time.time()
    wl = synth.make_workload(cfg, dev)
    torch.cuda.synchronize()
    log(f"[bench] {cfg.name}: inputs generated in {time.time() - t0:.1f}s "
        f"(keys {tuple(wl.keys.shape)} {wl.keys.dtype})")

    # ---- A by spherical K-means, index build (both timed, outside the step) ----
    km_ms, A, assign = kmeans_record(cfg, wl, dev)
    log(f"[bench] K-means ({cfg.kmeans_iters} iterations): {km_ms:.1f} ms; assignment alone: {assign}")
    ib, _ = index_build_record(cfg, wl, A, ws_bytes, dev, reps=20 if args.config == "c4" else 5, km_ms=km_ms,
                               assign=assign)
    build_ms, keys_per_s, build_path, fused_phases = ib["ms"], ib["keys_per_s"], ib["path"], ib.get("fused_phases_ms")
    log(f"[bench] index build: {build_ms:.2f} ms ({keys_per_s / 1e6:.1f} M keys/s), ready for the attention (with the "
        f"key-ordered copy of the lists) {ib['ready_for_attention_ms']:.2f} ms; phases {fused_phases}; selection on a "
        f"chunk of Y {ib['select_gbs']:.0f} GB/s; lists {ib['lists_bit_exact']}")
    mem = Memory.build(wl.keys, wl.values, A, Z, workspace_bytes=ws_bytes)

    # extending the index by M new keys instead of rebuilding it (same lists as a rebuild over N+M keys)
    append = None
    if N >= Z and wl.k_local is not None:
        idx_v, val_v = ops.build_index(A, wl.keys, Z, ws_bytes, return_values=True)
        append = {}
        for M in (1, wl.k_local.shape[1]):       # the local window's keys are the ones a memory takes in next
            K_new = wl.k_local[:, :M].contiguous()
            ms_copy, _ = timed(lambda: ops.index_append(A, K_new, N, idx_v, val_v, Z), reps=3, warm=1)
            i2, v2 = idx_v.clone(), val_v.clone()
            ops.index_append(A, K_new, N, i2, v2, Z, inplace=True)          # warm, on a copy of its own
            i2.copy_(idx_v), v2.copy_(val_v)
            ms_inpl, _ = timed(lambda: ops.index_append(A, K_new, N, i2, v2, Z, inplace=True), reps=1, warm=0)
            append[f"M={M}"] = {"out_of_place_ms": ms_copy, "in_place_ms": ms_inpl,
                               "rebuild_over_append": build_ms / ms_inpl}
            del i2, v2
        del idx_v, val_v
        log(f"[bench] index append: {append}")

    workload_name = (f"{cfg.name}: H={H} KV heads, G={G}, d={d}, N={N} keys/head, C={C}, Z={Z}, "
                     f"S={S} tokens/q-head ({H * Sq} query-heads)"
                     + (f", {wl.k_local.shape[1]} local keys causal + LSE merge" if wl.k_local is not None else ""))
    q = wl.queries
    # the lists as the attention reads them: Memory's copy in ascending key order (made once per index)
    ko_ms = ib["lists_key_order_ms"]
    attn_lists = mem.attention_lists(Sq) if args.list_order == "key" else mem.bucket_idx.reshape(-1)
    log(f"[bench] lists in key order: {ko_ms:.2f} ms (once per index); the step reads them in {args.list_order} order")
    has_local = wl.k_local is not None
    attn_events = []
    part_events = {"qhash": [], "group": [], "local": [], "merge": []}

    def step(record=True):
        e0, e1 = ev_pair()
        e0.record()
        qh = mem.hash(q)
        e1.record()
        g0, g1 = ev_pair()
        groups = ops.group_queries(qh, C)
        g1.record()
        a0, a1 = ev_pair()
        a0.record()
        mo, ml = ops.hash_attn_fwd(q, mem.keys, mem.values, attn_lists, mem.bucket_off,
                                   mem.bucket_cnt, groups, sm_scale)
        a1.record()
        if has_local:
            l1, m1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            lo, ll = ops.local_attn_fwd(q.reshape(H * G, S, d), wl.k_local, wl.v_local, sm_scale, True)
            l1.record()
            out, lse = update_out_and_lse(None, None, lo.reshape(H, Sq, d), ll.reshape(H, Sq))
            out, lse = update_out_and_lse(out, lse, mo, ml)
            m1.record()
        else:
            out, lse = mo, ml
        if record:
            attn_events.append((a0, a1))
            part_events["qhash"].append((e0, e1))
            part_events["group"].append((e1, g1))
            if has_local:
                part_events["local"].append((a1, l1))
                part_events["merge"].append((l1, m1))
        return out, lse, qh, groups, mo, ml

    settle(lambda: step(record=False))
    for _ in range(args.warmup):
        step(record=False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        res = step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    qheads = H * Sq
    value = qheads / (ms_per_step * 1e-3)
    out, lse, qh, groups, mo, ml = res
    query_path = {"ms_per_step": ms_per_step, "query_heads_per_s": value}
    if args.config == "c4":
        # index-build-heavy configuration: a step is one index build over all H*N keys
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            ops.build_index(A, wl.keys, Z, ws_bytes)
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        value = H * N / (ms_per_step * 1e-3)

    # ---- backward of the gathered attention (training use), timed beside the forward ----
    backward = None
    if not args.no_backward:
        dout = torch.randn_like(mo)
        dkb = torch.zeros(mem.keys.shape, dtype=torch.float32, device=dev)
        dvb = torch.zeros_like(dkb)
        run_bwd = lambda: ops.hash_attn_bwd(q, mem.keys, mem.values, attn_lists, mem.bucket_off,
                                            mem.bucket_cnt, groups, mo, ml, dout, sm_scale, dkb, dvb)
        bwd_ms, _ = timed(run_bwd, reps=2, warm=1)
        n_tiles = int(((groups.bin_count + 15) // 16).sum().item())       # 16-query tiles, each sweeps its bucket
        atomic_bytes = n_tiles * Z * 2 * d * 4
        backward = {"atomic": {"ms": bwd_ms,
                               "kernel": "hash_attn_bwd_mfma_kernel" if (d == 128 and e == 2)
                               else "hash_attn_bwd_generic_kernel",
                               "atomic_bytes_per_launch": atomic_bytes, "atomic_gbs": atomic_bytes / bwd_ms / 1e6}}
        log(f"[bench] backward of the gathered attention, atomic adds: {bwd_ms:.2f} ms "
            f"({backward['atomic']['atomic_gbs']:.0f} GB/s of atomic adds)")
        if d == 128 and e == 2:
            # without atomics: per-bucket partial rows + a sum per key over the inverted lists
            lists = attn_lists
            inv_ms, inv = timed(lambda: ops.inverse_index(lists, mem.bucket_off, mem.bucket_cnt, N), reps=1, warm=1)
            run_st = lambda: ops.hash_attn_bwd_staged(q, mem.keys, mem.values, lists, mem.bucket_off, mem.bucket_cnt,
                                                      groups, inv, mo, ml, dout, sm_scale, dkb, dvb)
            st_ms, _ = timed(run_st, reps=2, warm=1)
            hit = int((groups.bin_count > 0).sum().item())
            staged_bytes = hit * Z * (2 * d * e + 4) + 2 * hit * Z * 2 * d * e + 2 * H * N * d * 4 * 2
            backward["staged"] = {"ms": st_ms, "inverse_index_ms": inv_ms,
                                  "kernels": "hash_attn_bwd_staged_kernel + bwd_reduce_kernel",
                                  "algorithmic_bytes": staged_bytes, "gbs": staged_bytes / st_ms / 1e6,
                                  "hbm_frac": staged_bytes / st_ms / 1e6 / HBM_PEAK_GBS}
            log(f"[bench] backward without atomics: {st_ms:.2f} ms ({backward['staged']['gbs']:.0f} GB/s algorithmic; "
                f"inverse index of the lists, once per index: {inv_ms:.1f} ms)")
            del inv
        best = min(v["ms"] for v in backward.values())
        backward["ms"] = best
        backward["query_heads_per_s"] = qheads / (best * 1e-3)
        del dout, dkb, dvb

    attn_ms = sum(a.elapsed_time(b) for a, b in attn_events) / len(attn_events)
    parts_ms = {k: (sum(a.elapsed_time(b) for a, b in v) / len(v) if v else None) for k, v in part_events.items()}
    # algorithmic bytes of the gather-attention launch: every hit bucket once + q, out, lse
    hit = int((groups.bin_count > 0).sum().item())
    alg_bytes = hit * Z * (2 * d * e + 4) + qheads * (2 * d * e + 4)
    alg_flops = 4.0 * d * Z * qheads
    achieved = alg_bytes / attn_ms / 1e6
    attn_kernel = ops.hash_attn_fwd_kernel_name(H, Sq, N, d, C, cfg.dtype)     # what the library's dispatch took
    launches = ops.hash_attn_fwd_launches(H, Sq, N, d, C, cfg.dtype)           # one per row on large memories
    # fabric-side bytes per launch as the profiler counts them (L2 misses; HBM and the last-level cache answer)
    traffic = hbm_traffic(attn_kernel, cfg.name, required=args.config != "c1" and not args.head_dim)
    avg_launch_ms = attn_ms / launches
    hit_mask = groups.bin_count > 0
    rows_per_launch = H / launches
    distinct_rows = distinct_rows_per_launch(mem.bucket_idx, hit_mask, N)          # per row (KV head), averaged
    # what a launch must bring in from HBM at least once: the distinct K and V rows its hit buckets name, the
    # lists themselves, q, out and lse
    distinct_bytes = rows_per_launch * distinct_rows * 2 * d * e + (hit * Z * 4 + qheads * (2 * d * e + 4)) / launches
    roofline = {"kernel": attn_kernel,
                "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "algorithmic_over_hbm_peak": achieved / HBM_PEAK_GBS,
                "algorithmic_bytes_per_launch": alg_bytes / launches, "avg_launch_ms": avg_launch_ms,
                "launches_per_step": launches, "algorithmic_bytes_per_step": alg_bytes, "launches_ms_per_step": attn_ms,
                "hit_buckets": hit, "mfma_tflops": alg_flops / attn_ms / 1e9, "list_order": args.list_order,
                "distinct_rows_per_launch": rows_per_launch * distinct_rows,
                "distinct_bytes_per_launch": distinct_bytes}
    roofline["distinct_gbs"] = roofline["distinct_bytes_per_launch"] / avg_launch_ms / 1e6
    roofline["distinct_over_hbm_peak"] = roofline["distinct_gbs"] / HBM_PEAK_GBS
    roofline["reuse_factor"] = (alg_bytes / launches) / roofline["distinct_bytes_per_launch"]
    if traffic is not None:
        roofline["fabric_gbs"] = traffic / avg_launch_ms / 1e6
        roofline["fabric_probe_gbs"] = fabric_gather_probe(dev)
        # the same gather out of 2 MiB, which every L2 holds: what the path L2 -> compute unit gives scattered rows
        roofline["l2_gather_probe_gbs"] = fabric_gather_probe(dev, region_mib=2, passes=128)
        roofline["achieved_over_l2_gather_probe"] = roofline["achieved"] / roofline["l2_gather_probe_gbs"]
    if achieved > HBM_PEAK_GBS * 0.8 and traffic is not None:
        # Algorithmic bytes count a bucket's rows once per hit bucket; where every row is listed in many buckets
        # most of those requests are answered by an L2 or by the last-level cache, and algorithmic bytes / time
        # is not a rate any memory delivers.  The bounded figure: the L2 misses per second (fabric_gbs) over the
        # rate the path last-level cache -> L2 shows for scattered rows in the same run (fabric_probe_gbs).
        roofline["bound"] = "llc_fabric"
        roofline["frac"] = roofline["fabric_gbs"] / roofline["fabric_probe_gbs"]
        roofline["frac_is"] = ("fabric_gbs / fabric_probe_gbs (traffic per launch / avg_launch_ms over the gather "
                               "probe's rate); algorithmic_over_hbm_peak keeps achieved / peak")
        roofline["note"] = ("achieved = algorithmic bytes / time is not an HBM rate here: a key row listed in several "
                            "buckets comes from HBM once and from the last-level cache or an L2 for the others "
                            "(reuse_factor = algorithmic / distinct bytes); no_reuse_control is the same kernel where "
                            "nothing can be re-used.  Where the launches pace their sweeps (paced_sweeps) four of five "
                            "row requests are answered by an L2 and frac, the share of the fabric's rate the remaining "
                            "misses take, is well below 1: such a launch is bound by the latency of its loads with one "
                            "tile per wave in flight, not by a rate (l2_gather_probe_gbs: what the L2s give the same "
                            "row fetches when every one hits).  traffic is the average over a step's launches, "
                            "paced or not")
    log(f"[bench] step {ms_per_step:.2f} ms -> {value / 1e6:.2f} M {'keys/s' if args.config == 'c4' else 'query-heads/s'}"
        f"; attention kernel "
        f"{attn_ms:.2f} ms = {achieved:.0f} GB/s algorithmic ({100 * achieved / HBM_PEAK_GBS:.1f}% of HBM peak); "
        f"parts {parts_ms}")

    if attn_kernel.startswith("hash_attn_wave_kernel") and launches > 1:
        # where the schedules of the paced per-row launches stand (100 MHz ticks per key; see fastmem_debug.h)
        pace = [ops.wave_pace_state(N, C, Sq, attn_lists, r) for r in range(H)]
        roofline["paced_sweeps"] = {
            "rows_paced": sum(1 for p in pace if p["mode"] == 1),
            "rows_given_up": sum(1 for p in pace if p["mode"] == 2),
            "schedule_us_per_launch": [round(p["ticks_per_key"] * N / 100.0, 1) for p in pace],
            "unpaced_us_per_launch": [round(p["unpaced"] * N / 100.0, 1) for p in pace],
            "last_launch_us": [round(p["last_launch"] * N / 100.0, 1) for p in pace]}
        log(f"[bench] paced sweeps: {roofline['paced_sweeps']}")

    # read bandwidth a plain streaming-read kernel reaches on this device, for scale beside the published peak
    probe = torch.empty(4 << 30, dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    best_ms = min(timed(lambda: _lib.check(_lib.load().fm_debug_read(
        probe.data_ptr(), probe.numel(), sink.data_ptr(), torch.cuda.current_stream().cuda_stream)), reps=1, warm=1)[0]
        for _ in range(5))
    read_ceiling = probe.numel() / best_ms / 1e6
    del probe
    roofline["streaming_read_probe_gbs"] = read_ceiling
    roofline["vs_streaming_read_probe"] = achieved / read_ceiling
    log(f"[bench] streaming-read probe: {read_ceiling:.0f} GB/s; attention kernel at "
        f"{100 * achieved / read_ceiling:.1f}% of it")

    if not args.no_control:
        # the same launch over the lists in the other order (descending score, as torch.topk leaves them, is a
        # random key order), for scale
        other_lists = mem.bucket_idx.reshape(-1) if args.list_order == "key" else mem.attention_lists(Sq)
        other_ms = min(timed(lambda: ops.hash_attn_fwd(q, mem.keys, mem.values, other_lists, mem.bucket_off,
                                                       mem.bucket_cnt, groups, sm_scale), reps=2, warm=1)[0]
                       for _ in range(2))
        roofline["other_list_order"] = {"list_order": "value" if args.list_order == "key" else "key",
                                        "launch_ms": other_ms, "gbs": alg_bytes / other_ms / 1e6}
        log(f"[bench] the same launch over lists in {roofline['other_list_order']['list_order']} order: "
            f"{other_ms:.2f} ms")
    if not args.no_control and args.config == "c5":
        ctl = no_reuse_control(dev, list_order=args.list_order)
        roofline["no_reuse_control"] = ctl
        log(f"[bench] no-reuse control ({ctl['kernel']}): {ctl['launch_ms']:.2f} ms = {ctl['gbs']:.0f} GB/s "
            f"({100 * ctl['hbm_frac']:.1f}% of HBM peak) with every K/V row read once from HBM")

    if args.calibrate_copy:
        calibrate_copy(dev)

    # ---- CPU baseline on a bounded sample (head 0), also used as a parity spot check ----
    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        from oracle import cpu_path
        threads = cpu_threads()
        torch.set_num_threads(threads)
        K0, V0, A0 = wl.keys[0].cpu(), wl.values[0].cpu(), A[0].cpu()
        lists0 = mem.bucket_idx[0].cpu().long()
        q0 = q[0].cpu()
        kl0 = wl.k_local[0].cpu() if has_local else None
        vl0 = wl.v_local[0].cpu() if has_local else None
        pick = lambda m: torch.linspace(0, Sq - 1, m).long()        # spread over heads and positions
        # The sample: the queries of KV head 0 that fall into its first B buckets (the cost is per bucket
        # gathered, so the sample is sized in buckets).  A pilot over 8 buckets sizes B so that one pass takes
        # about a quarter of the budget; then one warm-up pass and three timed passes, median reported.
        qh0 = qh[0].cpu().long()
        pos0 = torch.arange(Sq) % S

        def one_pass(n_buckets):
            sel_q = (qh0 < n_buckets).nonzero().flatten()
            cpu_path.time_query_path(q0[sel_q], K0, V0, A0, lists0, sm_scale, kl0, vl0, pos0[sel_q], S)
            return int(sel_q.numel())

        tp0 = time.perf_counter()
        one_pass(min(C, 8))
        per_bucket = max((time.perf_counter() - tp0) / min(C, 8), 1e-6)
        B = int(max(min(C, 8), min(C, args.cpu_seconds / 4.0 / per_bucket)))
        n_sample = int((qh0 < B).sum())
        t_med, t_all = cpu_timed(lambda: one_pass(B), reps=3)
        sel = pick(min(Sq, 4096))                                      # parity spot-check sample of head 0
        # index-build sample: a few rows of A against all keys of head 0
        r = min(C, 32 if N > 200000 else 64)
        t_build, _ = cpu_timed(lambda: cpu_path.build_rows(A0[:r], K0, Z), reps=3 if N <= 300000 else 1)
        cpu = {"value": n_sample / t_med, "unit": "query-heads/s", "cores": threads, "kind": "port",
               "cpu_model": cpu_model(), "host_cpu_count": os.cpu_count(),
               "protocol": "1 warm-up pass + 3 timed passes, median",
               "pass_seconds": t_all,
               "sample": f"KV head 0: the {n_sample} query-heads that hash to its first {B} of {C} buckets, full "
                         f"N={N}, Z={Z}; hash + per-bucket gathered softmax attention"
                         + (" + causal local attention + merge" if has_local else ""),
               "index_build_rows_per_s": r / t_build,
               "index_build_keys_per_s_extrapolated": N / (C * t_build / r),
               "index_build_sample": f"{r} of {C} bucket rows of head 0 against all {N} keys, {t_build:.2f} s"}
        # parity spot check of the GPU results on the same sample
        co, cl, ch = cpu_path.hashed_attention(q0[sel], K0, V0, A0, lists0, sm_scale)
        gh = qh[0].cpu().long()[sel]
        same = gh == ch
        go, gl = mo[0].float().cpu()[sel], ml[0].cpu()[sel]
        parity = {"hash_agree_frac": same.float().mean().item(),
                  "out_max_abs_err": (go[same] - co[same]).abs().max().item(),
                  "lse_max_abs_err": (gl[same] - cl[same]).abs().max().item(),
                  "bucket_rows_bit_exact_vs_cpu_stable_sort_of_gpu_Y": None}
        Yg = ops.project(A[:1, :r].contiguous(), wl.keys[:1])[0].cpu()
        ref_lists = torch.sort(Yg + 0.0, dim=-1, descending=True, stable=True)[1][:, :min(Z, N)]
        parity["bucket_rows_bit_exact_vs_cpu_stable_sort_of_gpu_Y"] = bool(
            torch.equal(ref_lists, mem.bucket_idx[0, :r].cpu().long()))
        log(f"[bench] cpu baseline: {cpu['value']:.1f} query-heads/s on {threads} threads ({cpu['cpu_model']}), "
            f"passes {['%.2f' % t for t in t_all]} s; parity {parity}")

    if args.config == "c4" and ib.get("filter_roofline"):
        roofline = dict(ib["filter_roofline"], mfma_stream_probe_tflops=fused_phases["mfma_stream_probe_tflops"])

    # ---- the index-build half of the metric on the configuration it is quoted on (c4), in the same line ----
    index_build_c4 = None
    if args.config == "c5" and not args.no_c4_build:
        del mem, attn_lists, out, lse, qh, groups, mo, ml, res, q
        wl = None
        torch.cuda.empty_cache()
        cfg4 = synth.CONFIGS["c4"]
        t0 = time.time()
        wl4 = synth.make_workload(cfg4, dev)
        km4_ms, A4, assign4 = kmeans_record(cfg4, wl4, dev)
        index_build_c4, _ = index_build_record(cfg4, wl4, A4, ws_bytes, dev, reps=20, km_ms=km4_ms, assign=assign4)
        index_build_c4["workload"] = (f"{cfg4.name}: H={cfg4.H} KV heads, d={cfg4.d}, N={cfg4.N} keys/head, C={cfg4.C}, "
                                      f"Z={cfg4.Z}, A from {cfg4.kmeans_iters} K-means iterations on the keys")
        index_build_c4["fit_plus_build_ms"] = km4_ms + index_build_c4["ms"]
        log(f"[bench] c4 index build ({time.time() - t0:.1f} s wall with its inputs): {index_build_c4['ms']:.3f} ms = "
            f"{index_build_c4['keys_per_s'] / 1e9:.2f} G keys/s; K-means {km4_ms:.2f} ms; filter "
            f"{index_build_c4.get('filter_roofline')}; selection {index_build_c4['select_gbs']:.0f} GB/s; lists "
            f"{index_build_c4['lists_bit_exact']}")
        del wl4, A4

    line = {
        "metric": "index-build keys/s" if args.config == "c4" else "hashed-attn query-heads/s",
        "value": value, "unit": "keys/s" if args.config == "c4" else "query-heads/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if e == 2 else "f32", "data": "synthetic",
        "config": {"workload": workload_name,
                   "step": ("index build (sampled thresholds + fused MFMA filter + selection) over all keys"
                            if args.config == "c4" else
                            "qhash + group + gather attention" + (" + local attention + merge" if has_local else ""))},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "index_build": dict(ib, append=append),
        "index_build_c4": index_build_c4,
        "query_path": query_path,
        "step_parts_ms": {"attention": attn_ms, **parts_ms},
        "backward": backward,
        "parity_spot_check": parity,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
