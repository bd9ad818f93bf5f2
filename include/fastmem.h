/*
 * fastmem.h -- C ABI of libfastmem.so, the MI355X (gfx950) implementation of
 * the indexed-memory attention hot path of notbadai/fast_memory.
 *
 * The reference has no native boundary: its only operator is the torch custom
 * op `notbad::attention_hash_varlen` (triton_kernel.py:16-41) plus plain torch
 * calls around it.  Each entry point below names the reference lines whose work
 * it takes over.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the name ends in `_host`;
 *   - tensors are dense, row-major, batch-first: A [H,C,d], K/V [H,N,d],
 *     q/out [H,Sq,d] with Sq = G*S (query head hq = h*G + g, memory.py:281);
 *   - `dtype` selects the element type of q/k/v/A: FM_F32, FM_BF16 or FM_F16 (the
 *     reference's own performance harness runs fp16, triton_kernel.py:496); all
 *     accumulation is fp32; log-sum-exp values are fp32 natural logarithms;
 *   - all index tensors are int32;
 *   - `stream` is a hipStream_t (NULL = the default stream); no entry point
 *     synchronises the device or allocates memory; scratch space comes in
 *     through `ws` / `ws_bytes`, sized by the matching *_workspace() query;
 *   - return value: FM_OK (0) or an fm_status error code; fm_last_error()
 *     returns the message of the calling thread's last failure;
 *   - calls are re-entrant per stream as long as they do not share outputs or
 *     workspace (the switches of fastmem_debug.h are process-wide: a test that
 *     flips one must not run beside other callers).
 */
#ifndef FASTMEM_H
#define FASTMEM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  FM_OK = 0,
  FM_ERR_ARG = 1,         /* null pointer, bad extent, bad enum              */
  FM_ERR_UNSUPPORTED = 2, /* shape outside what the kernels are built for    */
  FM_ERR_WORKSPACE = 3,   /* ws_bytes smaller than the *_workspace() answer  */
  FM_ERR_LAUNCH = 4       /* HIP reported an error at launch                 */
} fm_status;

typedef enum { FM_F32 = 0, FM_BF16 = 1, FM_F16 = 2 } fm_dtype;

/* Longest list min(Z, N) the selection sorts inside LDS.  Longer lists are accepted by fm_argtopz_f32 and
 * fm_build_index (sorted in the workspace, markedly slower); fm_build_index_fused and fm_index_append take
 * lists up to FM_MAX_Z only. */
#define FM_MAX_Z 16384
/* Largest head dimension. */
#define FM_MAX_D 256
/* Queries one attention work item carries (tile of one (row,bucket) group). */
#define FM_QTILE 64

int fm_version(void);
const char* fm_last_error(void);

/* ---- a1: projection  Y[h,c,n] = sum_d A[h,c,d] K[h,n,d]  (fp32 out) --------
 * replaces einsum at memory.py:261 / triton_kernel.py:277.  bf16 inputs use
 * MFMA with fp32 accumulation.  Y is [H,C,N] with row stride `ldy` elements
 * (ldy >= N). */
int fm_project(const void* A, const void* K, float* Y, int H, int C, int N, int d,
               int64_t ldy, int dtype, void* stream);

/* ---- a2: arg-top-Z over every row of an fp32 matrix -------------------------
 * replaces torch.topk at memory.py:273 / triton_kernel.py:278.  Output row r =
 * the min(Z,N) indices of the largest entries of Y[r,:], ordered by value
 * descending then index ascending (the first Z entries of a stable descending
 * sort; -0 == +0; NaN is the largest).  Long rows with Z <= 8192 are read once
 * (a threshold from a 1/16 sample, then one collecting pass; a row the sample
 * misleads falls back to exact radix passes), others about four times; the
 * result is the same.  idx_out is [rows, min(Z,N)] int32;
 * val_out (may be NULL) receives the selected values in the same order (-0 as
 * +0): the lists' values are what fm_index_append needs to extend an index.
 * fm_argtopz_workspace is 0 unless min(Z, N) > FM_MAX_Z. */
size_t fm_argtopz_workspace(int64_t rows, int N, int Z);
int fm_argtopz_f32(const float* Y, int64_t rows, int N, int64_t ldy, int Z, int32_t* idx_out,
                   float* val_out, void* ws, size_t ws_bytes, void* stream);

/* ---- a1+a2: index build without handing Y to the caller ---------------------
 * memory.py:260-278 on one device.  idx_out [H,C,min(Z,N)] int32, val_out (may
 * be NULL) the projections of the listed keys, same shape, fp32.  The
 * workspace holds fp32 projection rows for as many (head,bucket) rows as fit;
 * any size from fm_build_index_workspace(...,1) up is accepted and larger ones
 * mean fewer passes. */
size_t fm_build_index_workspace(int H, int C, int N, int d, int Z, int64_t rows_per_pass);
int fm_build_index(const void* A, const void* K, int32_t* idx_out, float* val_out, int H, int C, int N,
                   int d, int Z, int dtype, void* ws, size_t ws_bytes, void* stream);

/* ---- a1+a2 fused: the same lists without ever writing Y to memory ------------
 * (memory.py:260-278; the selection sees exactly the fp32 values fm_project
 * would produce, so the lists are bit-identical to fm_build_index).  Built for
 * bf16 / fp16, d = 128, N >= 16384, 64 <= Z <= N/8; fm_build_index_fused_workspace
 * returns 0 for any other shape.  (It pays from about H * C * N = 2^24 on: 8 x
 * 256 x 32768 builds in 0.16 ms against 0.36 ms, 8 x 64 x 8192 in 0.095 ms
 * against 0.068 ms.)  A per-row threshold taken from a sample of the
 * keys filters the MFMA output; rows whose threshold missed are recomputed
 * exactly on the device (up to 64 of them).  status_dev (device,
 * FM_FUSED_STATUS_INTS ints) receives {rows repaired, rows left unresolved, then
 * the repaired rows as head * C + bucket, -1 in the unused places}; if the
 * second is non-zero the caller must rebuild with fm_build_index (until then the
 * unresolved rows list keys 0 .. Z-1: valid indices, not the right ones).  The
 * call reads nothing back: a caller may queue, or record into a graph, whatever
 * reads the lists behind it and look at the status word later. */
#define FM_FUSED_STATUS_INTS 66
size_t fm_build_index_fused_workspace(int H, int C, int N, int d, int Z, int dtype);
int fm_build_index_fused(const void* A, const void* K, int32_t* idx_out, float* val_out, int H, int C,
                         int N, int d, int Z, int dtype, void* ws, size_t ws_bytes, int32_t* status_dev,
                         void* stream);

/* ---- a3: query hash  h_q = argmax_c A[h,c,:].q  (first maximum wins) ---------
 * replaces einsum+argmax at memory.py:281-283 / triton_kernel.py:280-281.
 * hash_out [H,Sq] int32.  scores_out is optional ([H,Sq,C] fp32, may be NULL):
 * the scores the argmax was taken over. */
int fm_qhash(const void* A, const void* q, int32_t* hash_out, float* scores_out, int H, int C,
             int Sq, int d, int dtype, void* stream);

/* ---- a4: window filter of bucket lists -------------------------------------
 * memory.py:128-142: keep entries in [lo,hi), re-base by -lo, flatten row-major.
 * idx_in [H*C, Z]; idx_out holds up to H*C*Z entries; cnt_out/off_out [H*C]. */
size_t fm_window_filter_workspace(int64_t n_buckets_total);
int fm_window_filter(const int32_t* idx_in, int64_t n_buckets_total, int Z, int64_t lo, int64_t hi,
                     int32_t* idx_out, int32_t* cnt_out, int64_t* off_out, void* ws,
                     size_t ws_bytes, void* stream);

/* ---- exclusive prefix sum of per-bucket counts (triton_kernel.py:86-88) ----- */
int fm_bucket_offsets(const int32_t* cnt, int64_t n, int64_t* off_out, void* stream);

/* ---- a5 + a16: group queries by (row, bucket) on the device -----------------
 * replaces sort / unique_consecutive / cumsum at triton_kernel.py:75-88, with
 * no host synchronisation.
 *   q_hash    [H,Sq]   in   bucket of every query
 *   q_perm    [H,Sq]   out  stable ascending sort permutation per row:
 *                           q_perm[h,p] = original index of the p-th sorted query
 *   bin_count [H,C]    out  queries per bucket (memory.py:285-286)
 *   bin_off   [H,C]    out  first sorted position of the bucket, over the
 *                           flattened H*Sq axis (triton_kernel.py:84)
 *   items     [max_items] out  work items {row, bucket, first sorted position,
 *                           number of queries <= FM_QTILE}
 *   n_items   [1]      out  number of items written
 * max_items must be >= fm_group_max_items(H, C, Sq).  A query whose hash is outside
 * [0, C) belongs to no bucket: it is counted in no bin and is part of no item.  The
 * grouped queries of all rows fill the first T slots of q_perm (T = bin_off +
 * bin_count of the last bin); each query without a bucket leaves -(h*Sq + i) - 1 in
 * one of the H*Sq - T slots behind them (in no particular order), which is where the
 * attention entry points below find the rows that no work item writes. */
typedef struct { int32_t row, bucket, q_start, n_q; } fm_item;
int64_t fm_group_max_items(int H, int C, int Sq);
size_t fm_group_queries_workspace(int H, int C, int Sq);
int fm_group_queries(const int32_t* q_hash, int H, int C, int Sq, int32_t* q_perm,
                     int32_t* bin_count, int32_t* bin_off, fm_item* items, int32_t* n_items,
                     int64_t max_items, void* ws, size_t ws_bytes, void* stream);

/* ---- a6-a8: bucket-gathered attention forward ------------------------------
 * replaces the Triton kernel _attn_fwd/_attn_fwd_inner (triton_kernel.py:
 * 137-272) and the un-permute / unit conversion at triton_kernel.py:108-117.
 *   q [H,Sq,d], k,v [H,N,d]           in original order
 *   k_idx flat int32, bucket_off [H*C] int64, bucket_cnt [H*C] int32
 *   q_perm, items, n_items            from fm_group_queries
 *   out [H,Sq,d] (dtype of q), lse [H,Sq] fp32 natural log, original order.
 * A query whose bucket is empty gets out = 0, lse = -FLT_MAX, and so does a query
 * that is part of no item (hash outside [0, C), see fm_group_queries).
 * On large memories (bf16 / fp16, d = 128, K and V of all rows 512 MB or more, rows
 * of 2048 or more buckets that receive 24 queries or fewer each) the call is one
 * launch per row, which takes the row's work items in an order of its own (heavy
 * and light ones paired) and whose waves may sweep the row's key range on a common
 * schedule against the device's clock (lists in ascending key order are what this is
 * for: see fm_lists_key_order).  The library looks for the fastest schedule such a
 * launch keeps from call to call, per (N, C, Sq, k_idx, row), in a table of its own
 * in device memory (64 KB per GPU, no allocation; its address is asked for at the
 * first such call outside stream capture -- calls captured before that run unpaced),
 * and holds it only while it is faster than the launch left to itself; the first
 * calls on a memory can be slower than the settled ones (about 15).  Results do not
 * depend on the schedule or the order: the same bits paced and unpaced. */
int fm_hash_attn_fwd(const void* q, const void* k, const void* v, const int32_t* k_idx,
                     const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                     const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                     float* lse, int H, int Sq, int N, int d, int C, float sm_scale, int dtype,
                     void* stream);
/* The same with fm_hash_attn_fwd_workspace(max_items) bytes of device memory to work in (no counterpart in
 * the reference, whose launch grid is one program per 64 queries of a bucket, triton_kernel.py:99-106):
 * where buckets receive more than FM_QTILE queries on average a workgroup takes three items of a bucket
 * together, and with the workspace the groups are listed first so that every workgroup started has one --
 * without it two of three return at once, which leaves compute units idle (1.3 x slower at 128 queries per
 * bucket).  Same results bit for bit.  ws = NULL is fm_hash_attn_fwd; a workspace smaller than that is
 * refused (FM_ERR_WORKSPACE). */
size_t fm_hash_attn_fwd_workspace(int64_t max_items);
int fm_hash_attn_fwd_ws(const void* q, const void* k, const void* v, const int32_t* k_idx,
                        const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                        const fm_item* items, const int32_t* n_items, int64_t max_items, void* out,
                        float* lse, int H, int Sq, int N, int d, int C, float sm_scale, int dtype,
                        void* ws, size_t ws_bytes, void* stream);

/* ---- lists in ascending key order, for the gathered attention ------------------
 * The kernel of triton_kernel.py:230-272 walks a bucket's list in stored order, and
 * softmax(q.K^T).V over a list does not depend on that order (only the rounding of
 * the fp32 sums does).  torch.topk (memory.py:273) leaves the lists in descending
 * score order, which is a random key order; in ascending key order a 64-key tile
 * reads neighbouring pages of K and V, which makes fm_hash_attn_fwd and the
 * backward 10-20 % faster where many queries are served per build (nothing to gain
 * for a single query per row).  Same flat layout in and out (bucket_off,
 * bucket_cnt as for fm_hash_attn_fwd, n_lists of them; k_idx_out != k_idx); any
 * list length.  A list that names a key twice or a key outside [0, N) is copied
 * unchanged; n_unsorted [1] (device, may be NULL) receives the number of such
 * lists.  The value-ordered lists stay the ones fm_index_append extends. */
int fm_lists_key_order(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt,
                       int64_t n_lists, int N, int32_t* k_idx_out, int32_t* n_unsorted, void* stream);

/* ---- f1: backward of the bucket-gathered attention --------------------------
 * replaces ring_attention_masked_backward (memory.py:166-206), which forms the
 * dense [S, N] probability matrix; here only a query's bucket is visited.
 *   q, k, v, k_idx, bucket_off, bucket_cnt, q_perm, items, n_items, max_items
 *                                      as for fm_hash_attn_fwd
 *   out [H,Sq,d], lse [H,Sq] fp32      the forward's result, or the result merged
 *                                      with further keys (the gradients are then
 *                                      the gathered keys' share)
 *   dout [H,Sq,d]                      gradient of the loss w.r.t. out
 *   dlse [H,Sq] fp32, may be NULL      gradient of the loss w.r.t. lse (a caller that merges
 *                                      partial results by their lse outside has one; NULL = 0)
 *   dq [H,Sq,d] (dtype of q)           written; a query whose bucket is empty, or that has no
 *                                      bucket (hash outside [0, C)), gets 0
 *   dk, dv [H,N,d] fp32                ACCUMULATED into (atomic adds): zero them
 *                                      before the first call; several calls
 *                                      (key windows) may add into the same buffers.
 * The order of the atomic adds depends on scheduling, so the last bits of dk and
 * dv can differ between runs. */
int fm_hash_attn_bwd(const void* q, const void* k, const void* v, const int32_t* k_idx,
                     const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                     const fm_item* items, const int32_t* n_items, int64_t max_items, const void* out,
                     const float* lse, const void* dout, const float* dlse, void* dq, float* dk, float* dv, int H,
                     int Sq, int N, int d, int C, float sm_scale, int dtype, void* stream);

/* ---- f1, dense query sets: backward without atomics ---------------------------
 * Same gradients as fm_hash_attn_bwd (bf16 or fp16, d = 128 only; the partial rows
 * are bf16 for both).  A key's dk and dv rows
 * collect contributions from every bucket that lists it; here each (row, bucket)
 * workgroup writes the bucket's own partial rows (bf16, one per listed key, in the
 * workspace) and a second kernel sums, per key, the partial rows of the list
 * positions that name it -- full-line stores and loads in place of fp32 atomic
 * read-modify-writes, and a fixed summation order (results do not depend on
 * scheduling; only the first 256 queries of a bucket go through its partial
 * rows, a bucket that receives more adds the rest with fp32 atomic adds).  Pays when most buckets receive queries: a bucket without queries
 * still costs its rows (written as zeros and read back).
 *
 * fm_inverse_index: the inverse of the lists, which depends on the lists only and
 * can be kept with them (lists in any order: a stable radix sort of (key, position) pairs).  T = number of list entries (the sum of bucket_cnt, the
 * length of k_idx; row-major (row, bucket) order as everywhere).
 *   key_off [H*N + 1] int32   entries of key (h, n): sorted positions
 *                              key_off[h*N + n] .. key_off[h*N + n + 1]
 *   inv_pos [T] int32          flat list positions, ordered by (row, key, position)
 * fm_hash_attn_bwd_staged: q_perm, bin_off, bin_count from fm_group_queries;
 * row_pos_host [H+1] (HOST memory) = flat list position where each row's lists
 * begin (row_pos_host[H] = T); rows are processed in groups whose partial rows
 * (512 bytes per list entry) fit the workspace, which must hold at least the
 * longest row (fm_hash_attn_bwd_staged_workspace(entries of that row)).
 * dq is written, dk and dv (fp32) are accumulated into, as in fm_hash_attn_bwd. */
size_t fm_inverse_index_workspace(int64_t T, int H, int N);
int fm_inverse_index(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt, int H,
                     int C, int N, int64_t T, int32_t* key_off, int32_t* inv_pos, void* ws, size_t ws_bytes,
                     void* stream);
/* The same index without a sort, for lists in strictly ascending key order (every list as
 * fm_lists_key_order leaves it, no key twice): a transposition by key ranges, several times
 * faster (H, C <= 65535).  n_bad [1] (device) receives 0 when every list is in that order with
 * all keys in [0, N), and a positive count otherwise: then key_off / inv_pos hold no index
 * (every access still stays inside the buffers, and the call costs one pass over the lists)
 * and fm_inverse_index is the one to call.  Workspace: two tables of H*C*(N/256+1) words. */
size_t fm_inverse_index_key_order_workspace(int H, int C, int N);
int fm_inverse_index_key_order(const int32_t* k_idx, const int64_t* bucket_off, const int32_t* bucket_cnt, int H,
                               int C, int N, int64_t T, int32_t* key_off, int32_t* inv_pos, int32_t* n_bad,
                               void* ws, size_t ws_bytes, void* stream);
size_t fm_hash_attn_bwd_staged_workspace(int64_t max_row_entries);
int fm_hash_attn_bwd_staged(const void* q, const void* k, const void* v, const int32_t* k_idx,
                            const int64_t* bucket_off, const int32_t* bucket_cnt, const int32_t* q_perm,
                            const int32_t* bin_off, const int32_t* bin_count, const void* out,
                            const float* lse, const void* dout, const float* dlse,
                            const int32_t* key_off, const int32_t* inv_pos, void* dq, float* dk,
                            float* dv, int H, int Sq, int N, int d, int C, const int64_t* row_pos_host,
                            float sm_scale, int dtype, void* ws, size_t ws_bytes, void* stream);

/* ---- the reference operator in one call -------------------------------------
 * attention_hash_varlen(q,k,v,k_hashes,k_hash_counts,q_hashes,sm_scale)
 * (triton_kernel.py:51-119): bucket offsets + grouping + attention.  A query whose
 * hash is outside [0, C) (the reference would fail on the index) is treated as
 * hashed to an empty bucket: out = 0, lse = -FLT_MAX. */
size_t fm_attention_hash_varlen_workspace(int H, int C, int Sq);
int fm_attention_hash_varlen(const void* q, const void* k, const void* v, const int32_t* k_idx,
                             const int32_t* bucket_cnt, const int32_t* q_hash, void* out,
                             float* lse, int H, int Sq, int N, int d, int C, float sm_scale,
                             int dtype, void* ws, size_t ws_bytes, void* stream);

/* ---- the same operator for callers that cannot allocate ------------------------
 * No counterpart in the reference.  For callers that cannot obtain device memory
 * for a workspace: code under HIP graph capture, tight serving loops, harnesses
 * that forbid allocation.  Identical to fm_attention_hash_varlen (same kernels,
 * same results bit for bit) except that the grouping tables, the query
 * permutation and the work items live in a device array of the library itself,
 * FM_STATIC_SCRATCH_BYTES long, which every GPU the library runs on holds until
 * the process ends.  The call allocates nothing and frees nothing; the first call
 * on a device looks the array's address up (hipGetSymbolAddress).  Extents whose
 * fm_attention_hash_varlen_workspace(H, C, Sq) exceeds FM_STATIC_SCRATCH_BYTES are
 * refused with FM_ERR_WORKSPACE.  All calls on one GPU share that GPU's array:
 * calls that overlap on one GPU (different streams or threads) race; successive
 * calls on one stream do not (each clears what it needs to start at zero with a
 * fill kernel, not a memset node). */
#define FM_STATIC_SCRATCH_BYTES (32u << 20)
int fm_attention_hash_varlen_static(const void* q, const void* k, const void* v, const int32_t* k_idx,
                                    const int32_t* bucket_cnt, const int32_t* q_hash, void* out,
                                    float* lse, int H, int Sq, int N, int d, int C, float sm_scale,
                                    int dtype, void* stream);

/* ---- decode batch over memories of different sizes ---------------------------
 * The same path (query hash memory.py:281-283 + gathered attention
 * triton_kernel.py:137-272) for a batch of rows whose memories differ in N, C
 * and Z -- one row = one KV head of one sequence, G <= 16 queries per row (the
 * G query heads of that KV head, one token each).  A, K, V of all rows are
 * packed back to back ([sum C, d], [sum N, d]); the bucket lists likewise, each
 * row holding C*Z indices local to its own keys.  bf16, d = 128 only.
 *   q [rows,G,d] -> out [rows,G,d], lse [rows,G] fp32, hash_out [rows,G] int32
 *   (required: a first launch hashes every row into it, a second reads it);
 *   scores_out (optional, [sum C, G] fp32): the scores the hashes were taken over. */
typedef struct {
  int64_t a_off;        /* first row of this row's A in A_all            */
  int64_t k_off;        /* first key row in K_all / V_all                */
  int64_t idx_off;      /* first element of its bucket lists in idx_all  */
  int32_t n_keys, n_buckets, bucket_size;
  int32_t q_row1;       /* 0: this row's queries are row i of q/out/lse/hash_out, i = position of the
                           descriptor; else they are row q_row1 - 1 (descriptors may then come in any
                           order, e.g. longest lists first so that the launch ends evenly)            */
} fm_rowdesc;
int fm_decode_hash_attn(const void* q, const void* A_all, const void* K_all, const void* V_all,
                        const int32_t* idx_all, const fm_rowdesc* desc, int rows, int G, int d,
                        float sm_scale, void* out, float* lse, int32_t* hash_out, float* scores_out,
                        int dtype, void* stream);

/* ---- a11: dense local attention with LSE ------------------------------------
 * the attention_forward(q,k_self,v_self,sm_scale,True) call at memory.py:302
 * (the reference ships no definition).  q [H*G,S,d], k,v [H,L,d]; causal is
 * bottom-right aligned: query i sees keys j <= i + (L - S). */
int fm_local_attn_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int H,
                      int G, int S, int L, int d, float sm_scale, int causal, int dtype,
                      void* stream);

/* ---- a10: LSE merge, in place on the running pair ---------------------------
 * update_out_and_lse (memory.py:54-71).  out [Q,d] fp32 and lse [Q] fp32 are
 * updated with block_out [Q,d] (dtype) and block_lse [Q] fp32. */
int fm_lse_merge(float* out, float* lse, const void* block_out, const float* block_lse, int64_t Q,
                 int d, int dtype, void* stream);

/* ---- a12/a13: construction of A ----------------------------------------------
 * fm_l2_normalize: rows / max(norm, eps)        (memory.py:214-217)
 * fm_topk_mean:    gather + mean + normalise    (memory.py:224-229, 258)
 *                  Xn [HG,N,d]; top_idx [C,HG,k] int32; A_out [C,H,d]
 * fm_segment_mean: spherical K-means centroid update (README.md:41-43):
 *                  X [H,N,d] unit rows, perm/seg_off/seg_cnt from
 *                  fm_group_queries on the labels; an empty cluster keeps
 *                  prev; cent_out [H,C,d] in dtype, unit rows.
 * fm_segment_mean_directions: the same update on rows of any length: member x
 *                  contributes x / max(||x||, eps), so K-means on the L2-normalised
 *                  keys (README.md:33-45) never stores the normalised copy (the
 *                  assignment argmax_c c.x does not depend on ||x||). */
int fm_l2_normalize(const void* X, void* Xn, int64_t rows, int d, float eps, int dtype,
                    void* stream);
int fm_topk_mean(const void* Xn, const int32_t* top_idx, void* A_out, int C, int H, int G, int N,
                 int k, int d, int normalize, int dtype, void* stream);
int fm_segment_mean(const void* X, const int32_t* perm, const int32_t* seg_off,
                    const int32_t* seg_cnt, const void* prev, void* cent_out, int H, int C, int N,
                    int d, int dtype, void* stream);
int fm_segment_mean_directions(const void* X, const int32_t* perm, const int32_t* seg_off,
                               const int32_t* seg_cnt, const void* prev, void* cent_out, int H, int C,
                               int N, int d, float eps, int dtype, void* stream);

/* ---- f3: extending an index by new keys -----------------------------------
 * The reference rebuilds the bucket lists from all keys on every forward
 * (memory.py:252-278); this merges M new keys (global indices n_old ..
 * n_old+M-1) into existing lists, with the result a rebuild over all n_old+M
 * keys would give, in O(Z + M) per bucket.
 *   A [H,C,d], K_new [H,M,d]
 *   idx_in, val_in  [H,C,min(Z,n_old)]      lists and their projections (val_out of
 *                                            the build or of an earlier append)
 *   idx_out, val_out [H,C,min(Z,n_old+M)]   either separate buffers, or exactly
 *                                            idx_in and val_in (in place; full lists
 *                                            only, n_old >= Z): a bucket that takes no
 *                                            new key is then not touched, so a few new
 *                                            keys cost almost no memory traffic
 *   status_dev (device, 1 int)               number of rows that accepted more new keys
 *                                            than the merge holds (8192): if non-zero the lists written are
 *                                            incomplete (in place: damaged), rebuild.
 * The workspace holds the fp32 projections of the new keys. */
size_t fm_index_append_workspace(int H, int C, int M);
int fm_index_append(const void* A, const void* K_new, int n_old, int M, const int32_t* idx_in,
                    const float* val_in, int32_t* idx_out, float* val_out, int H, int C, int Z, int d,
                    int dtype, void* ws, size_t ws_bytes, int32_t* status_dev, void* stream);

/* ---- f2: scatter-add of rows onto index lists -------------------------------
 * the segmented form of centroids.scatter_add_(...) in calc_ref_centroids
 * (memory.py:449-450): sum_out[h,c,:] = sum of X[h, perm[j], :] over the members j
 * of segment (h,c) (perm/seg_off/seg_cnt from fm_group_queries on the target
 * indices), fp32, in member order; an empty segment gives zeros. */
int fm_segment_sum(const void* X, const int32_t* perm, const int32_t* seg_off, const int32_t* seg_cnt,
                   float* sum_out, int H, int C, int N, int d, int dtype, void* stream);

/* Test and measurement hooks (fm_debug_*, fm_hash_attn_fwd_kernel) are declared in fastmem_debug.h: they are
 * process-wide switches and probes, not part of what a production caller binds. */

#ifdef __cplusplus
}
#endif
#endif /* FASTMEM_H */
