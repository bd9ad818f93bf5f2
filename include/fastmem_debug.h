/*
 * fastmem_debug.h -- test and measurement hooks of libfastmem.so.
 *
 * None of these has a counterpart in the reference.  The switches take effect only in a process whose
 * environment held FASTMEM_DEBUG_HOOKS=1 when the library was first called (fm_debug_hooks_enabled() says
 * whether it did); in any other process the setters do nothing, so no caller can reroute another caller's
 * kernels.  The switches (fm_debug_force_generic,
 * fm_debug_argtopz_exact_only, fm_debug_fused_filter, fm_debug_set_phase_events) are PROCESS-WIDE state, read by every call on
 * every stream: they exist so that tests can compare two implementations of one operator and so that the
 * benchmark can time the phases of the fused build; a production caller never touches them.  The probes
 * (fm_debug_copy, fm_debug_read, fm_debug_gather, fm_debug_mfma) are plain kernels of known size.
 */
#ifndef FASTMEM_DEBUG_H
#define FASTMEM_DEBUG_H

#include "fastmem.h"

#ifdef __cplusplus
extern "C" {
#endif

/* 1 if the switches below take effect in this process (FASTMEM_DEBUG_HOOKS=1 at the first call), else 0. */
int fm_debug_hooks_enabled(void);

/* Diagnostic: 1 routes the attention entry points through the generic kernels
 * (used by tests to compare the two implementations), 0 restores dispatch.  For
 * fm_hash_attn_fwd on bf16 / fp16, d = 128 only: 2 = always the kernel that stages a
 * bucket's rows in LDS, one work item per workgroup, in a single launch, 6 = the
 * same in one launch per row; 4 = the staged kernel with two work items per
 * workgroup; 5 = always the kernel that loads the rows straight into LDS (three
 * items per workgroup), in a single launch, 7 = the same in one launch per row;
 * 3 = always the kernel that gathers the rows into registers; 8 = the kernel of the
 * head dimensions 64 and 256 instantiated for 128 (tests compare it with the kernels
 * built for 128); 9 = (backward) the two-tile pass of fm_hash_attn_bwd_staged
 * loads its key blocks into registers as its other passes do, instead of through
 * LDS a block ahead (tests compare the two, which give the same bits); 10 = the
 * kernel with a wave per work item, launched as dispatch would launch it, 11 = that
 * kernel in a single launch, 12 = in one launch per row, 13 = the same with its
 * sweeps unpaced.  Dispatch: gather
 * when H min(Sq, C) < 512 and Sq < 24 C; else the direct loads up to 2^24 keys and
 * the staged kernel beyond; one launch per row when K and V of all rows are 512 MB
 * or more, those of a row 32 MB or more, and a row has 1024 (staged kernel: 1536)
 * or more buckets and queries; where the launches go per row, a row has 2048 or
 * more buckets and queries and a bucket receives 24 queries or fewer on average,
 * the kernel with a wave per work item in place of the direct loads. */
void fm_debug_force_generic(int on);

/* Diagnostic: where the schedule of the paced launches of "hash_attn_wave_kernel" stands for row `row` of a
 * memory of N keys, C buckets, Sq queries per row and the lists at k_idx (device pointer, as passed to
 * fm_hash_attn_fwd): out8 = { mode (0 measuring, 1 paced, 2 given up for a while), then in 100 MHz ticks per key:
 * the next launch's schedule, the fastest schedule kept in the current search, the mean of the launches on the
 * held schedule, the unpaced launch; launches the hold still lasts; ticks per key of the last launch and of its
 * schedule }; zeros before the first launch.  Copies from the device (synchronous). */
int fm_debug_wave_pace_state(int N, int C, int Sq, const void* k_idx, int row, float* out8);

/* Diagnostic: name of the kernel fm_hash_attn_fwd launches for these extents
 * (a static string): "hash_attn_generic_kernel", "hash_attn_wave_kernel" (a wave per work item),
 * "hash_attn_mfma_kernel" (rows
 * gathered into registers), "hash_attn_staged_kernel<1>" or "...<2>" (rows staged
 * in LDS through registers, one or two work items per workgroup),
 * "hash_attn_ring_kernel" (rows loaded straight into LDS, three work items per
 * workgroup); ", f16>" / "<f16>" marks the fp16 forms, "64-bit rows" the form for
 * memories of more than 2^24 keys.  bench.py names its roofline kernel with it. */
const char* fm_hash_attn_fwd_kernel(int H, int Sq, int N, int d, int C, int dtype);

/* Diagnostic: name of the kernel fm_local_attn_fwd launches for these extents (a static
 * string): "local_attn_dense_kernel<bf16|f16, 64|128|256>" (MFMA, a workgroup per 128
 * queries of a head), "local_attn_decode_kernel" (bf16, d = 128, one query per head) or
 * "local_attn_generic_kernel" (fp32 and other head dimensions). */
const char* fm_local_attn_fwd_kernel(int G, int S, int L, int d, int dtype);

/* Diagnostic: number of launches of that kernel one fm_hash_attn_fwd call makes for
 * these extents: 1, or H where the kernel goes out once per row (see above).  bench.py
 * divides its event time and the algorithmic bytes by it. */
int fm_hash_attn_fwd_launches(int H, int Sq, int N, int d, int C, int dtype);

/* Diagnostic: name of the filter kernel fm_build_index_fused launches for these
 * extents (a static string): "fused_filter_kernel" (four waves over a slab of 256
 * buckets) or "fused_filter_wide_kernel" (eight waves over a slab of 1024); NULL
 * where the fused build does not take the shape. */
const char* fm_build_index_fused_kernel(int H, int C, int N, int d, int Z, int dtype);

/* Diagnostic: 1 makes fm_argtopz_f32 (and the chunked index build) take the exact
 * multi-pass selection for every row instead of the sampled one-pass form (tests
 * compare the two), 0 restores dispatch. */
void fm_debug_argtopz_exact_only(int on);

/* Diagnostic: 1 keeps the fused index build away from the filter kernel that issues its epilogue between its
 * MFMAs (fused_filter_ping_kernel), so that it takes fused_filter_wide_kernel where it would take that one
 * (tests compare the lists of the two); 2, 3, 4 make it take that kernel, where the plan allows it, in the form
 * whose straight-line emission covers 64, 128 or 192 candidates of a group of 16 keys x 128 buckets (the plan picks
 * the form by the expected number; every form gives the same lists); 0 restores the plan. */
void fm_debug_fused_filter(int form);

/* Diagnostic: hand the fused index build up to 5 hipEvent_t (host array that
 * must stay valid; NULL clears) which it records on its stream before phase 0
 * (thresholds), 1 (MFMA filter), 2 (selection), 3 (repair) and at the end. */
void fm_debug_set_phase_events(void** events, int n);

/* Diagnostic: streaming copy of nbytes (multiple of 16) device to device; the
 * known-size kernel that profiler HBM counters are calibrated against. */
int fm_debug_copy(void* dst, const void* src, int64_t nbytes, void* stream);

/* Diagnostic: read-only stream over nbytes (multiple of 32768) of device memory;
 * nothing is written (sink: 4 bytes of device memory, left untouched).  Times the
 * read bandwidth a kernel reaches on the device. */
int fm_debug_read(const void* src, int64_t nbytes, void* sink, void* stream);

/* Diagnostic: `passes` sweeps over region_bytes (256 x a power of two >= 2^10) of device memory in which every
 * 256-byte row is read exactly once per sweep, in a scattered order, by sixteen lanes with a 16-byte load each
 * (the row fetch of the gathered attention); from one sweep to the next a row's reader moves behind another L2.
 * (A sweep is 2^17 rows at least: a region of fewer rows is read 2^17 / rows times per sweep, and the bytes a call
 * reads are passes * max(region_bytes, 32 MiB).  With a region that every L2 holds, 1 or 2 MiB, the rate is that
 * of the path from an L2 into the compute units for scattered rows.)
 * With a region that the last-level cache holds and an L2 does not (say 64 MiB), the bytes of every sweep after the
 * first come out of the last-level cache: region_bytes * passes / time is the rate the path from that cache into
 * the L2s sustains for scattered rows.  Nothing is written (sink: 4 bytes, left untouched). */
int fm_debug_gather(const void* src, int64_t region_bytes, int passes, void* sink, void* stream);

/* Diagnostic: a register-resident stream of v_mfma_f32_32x32x16_bf16 (no memory, LDS or VALU work in
 * the loop) over the first 5120 bf16 values at `operands` (n_operands >= 5120): iters * 2^33 flops per call.
 * Times the rate the matrix pipes sustain on the device for those operand values (the device clocks such a
 * loop lower the more the operand bits toggle).  sink: 4 bytes of device memory, left untouched. */
int fm_debug_mfma(const void* operands, int64_t n_operands, int iters, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTMEM_DEBUG_H */
