/*
 * mlora.h -- C ABI of libmlora_hip.so: multi-LoRA batched apply on MI355X (gfx950).
 *
 * The library replaces, for the LoRA-apply path only, what the reference reaches
 * through two foreign interfaces:
 *   - the third-party `punica.ops.add_lora_bgmv(y, x, wa_T_all, wb_T_all, indicies,
 *     layer_idx, scale)` CUDA op called from lightllm/models/lora_gpu.py:138,150,162
 *     (decode), and the `torch.bmm(torch.bmm(x, A), B)` pair at lora_gpu.py:127-128,
 *     145-146,157-158 (prefill);
 *   - nothing else: the copy helpers of the reference's own native module
 *     (csrc/interface.cpp:18-79) belong to the CPU-assisted transport, not to this path.
 *
 * Conventions
 *   - Every pointer named "device" is HIP device memory owned by the caller; the
 *     library keeps no pointer between calls and allocates nothing.
 *   - Calls are asynchronous on `stream` (a hipStream_t passed as void*, 0 = the
 *     null stream) and may be captured into a HIP graph.
 *   - 16-bit floats: dtype MLORA_F16 (IEEE binary16) or MLORA_BF16 (bfloat16);
 *     all products are accumulated in fp32 and rounded once (nearest even) on store.
 *   - Return value: MLORA_OK or a negative MLORA_E* code; mlora_last_error() then
 *     returns a thread-local message.  Nothing throws or exits.
 *   - Index validation that needs device data (adapter ids, page ids, ranks) is done
 *     inside the kernels: an out-of-range adapter id is treated as "no adapter" and
 *     counted in counters[MLORA_CNT_BAD]; an out-of-range page id contributes zero.
 *     No kernel reads or writes outside the extents given here.
 *
 * Paged adapter pool (one slab per layer, projection and side)
 *   rows      : [n_pages * page_rows, H] 16-bit floats, row-major, H % 8 == 0,
 *               base 16-byte aligned.  An A slab holds rank rows of A^T (length Hin),
 *               a B slab holds rank rows of B (length Hout).
 *   page_tbl  : int32 [n_adapters, max_pages]; rank row j of adapter i is row
 *               page_tbl[i][j / page_rows] * page_rows + j % page_rows, in the A slab and in the
 *               B slab alike (one table serves every layer, projection and side).
 *               page_rows is a power of two (1..64).
 *   rank      : int32 [n_adapters], 1..max_rank (max_rank <= 64).
 *   scaling   : float [n_adapters]  (alpha / r).
 *   tok_adapter : int32 [T]; a negative value means the token has no adapter.
 */
#ifndef MLORA_H
#define MLORA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLORA_OK 0
#define MLORA_EINVAL (-1)   /* bad size / null pointer / unsupported combination */
#define MLORA_ERANGE (-2)   /* value outside the supported range (rank, T, n_proj ...) */
#define MLORA_EALIGN (-3)   /* pointer or row width not 16-byte aligned */
#define MLORA_EDTYPE (-4)   /* dtype is neither MLORA_F16 nor MLORA_BF16 */
#define MLORA_ELAUNCH (-5)  /* the HIP runtime refused the launch */
#define MLORA_ENOSPACE (-6) /* caller-provided workspace too small */

#define MLORA_F16 0
#define MLORA_BF16 1

#define MLORA_MAX_PROJ 8      /* projections batched in one decode launch */
#define MLORA_MAX_RANK 64
#define MLORA_GATHER_MAX_T 8192   /* tokens one mlora_pool_gather call can group */

/* counters[] written by mlora_pool_gather (device int32[8]) */
#define MLORA_CNT_NSEG 0     /* number of segments (distinct adapters present) */
#define MLORA_CNT_NVALID 1   /* tokens that have an adapter */
#define MLORA_CNT_NCHUNK 2   /* decode work items (chunks of <= group tokens of one adapter) */
#define MLORA_CNT_BAD 3      /* tokens whose adapter id was >= n_adapters (treated as none) */
#define MLORA_CNT_WORDS 8

/* Decode work records written by mlora_pool_gather and read by mlora_bgmv_multi: one record of
 * MLORA_WORK_WORDS int32 per workgroup and projection, MLORA_WORK_CAP(T) records per batch. */
#define MLORA_WORK_WORDS 80
#define MLORA_WORK_CAP(T) ((((T) + 7) / 8) * 8)

const char *mlora_last_error(void);
int mlora_version(void);

/*
 * Adapter-pool index/offset gather + grouping of tokens by adapter.
 * Replaces the per-token index vector the reference draws at lora_gpu.py:120 and
 * selects at :124,143,155 (and the unused real ids of pre_process.py:50,100).
 *
 * Per-token view (each output may be NULL to skip it):
 *   out_row_off [T, max_pages] = page_tbl[a][p] * page_rows for p < ceil(rank[a]/page_rows), else -1
 *   out_rank [T], out_scale [T]                      (0 / 0.0f for tokens without adapter)
 * Grouped view (all of perm..counters NULL to skip):
 *   perm [T]            token ids ordered by (adapter, token id); tokens without adapter last
 *   seg_start/len/adapter [min(T, n_adapters)]   runs of equal adapter, ascending adapter id
 *   chunk_start/len/adapter [T]   each segment cut into pieces of <= group tokens, then the
 *                       adapter-less tokens in pieces of <= group with adapter -1
 *   counters [MLORA_CNT_WORDS]
 *   work [MLORA_WORK_CAP(T) * MLORA_WORK_WORDS]  (optional, may be NULL) the chunks as decode work
 *                       records in launch order: position c of the chunk list is record
 *                       (c mod P) * 8 + c / P with P = ceil(n_chunks / 8): the records in use come first,
 *                       records b, b + 8, ... hold a range of P consecutive chunks (the one-launch decode
 *                       form runs such a range on one XCD; the two-launch form takes the records in
 *                       order).  For T <= 2048 the chunks of each such range are placed by falling rank
 *                       (ties in chunk order), which starts the workgroups of wide items first; the
 *                       chunk_* arrays keep chunk order.  Record words:
 *                       [0] tokens (0 = empty record) [1] adapter [2] rank [3] scaling (float bits)
 *                       [4..11] token ids [12..15] 0 [16..79] row of rank row j in a rows slab, -1 if
 *                       j >= rank or the page id is outside [0, n_pages).
 * T <= MLORA_GATHER_MAX_T.  All outputs are exact integers / copied floats (bit-exact).
 */
int mlora_pool_gather(const int32_t *tok_adapter, int T,
                      const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                      int n_adapters, int max_pages, int page_rows, int64_t n_pages,
                      int32_t *out_row_off, int32_t *out_rank, float *out_scale,
                      int32_t *perm, int32_t *seg_start, int32_t *seg_len, int32_t *seg_adapter,
                      int32_t *chunk_start, int32_t *chunk_len, int32_t *chunk_adapter, int group,
                      int32_t *counters, int32_t *work, void *stream);

/*
 * Adapter swap-in, device side: place rank rows that arrived from the host as contiguous blocks on
 * the pages an adapter owns.  For job j (one (layer, projection, side)): src[j] is [rank, row_elems[j]]
 * contiguous, dst_slab[j] the rows slab it belongs to; rank row k goes to slab row
 * pages[k / page_rows] * page_rows + k % page_rows.  `pages` is a HOST array of the slot's page ids.
 * Replaces the per-layer whole-tensor copies of the reference's swapper (shared_tensor.py:117-147)
 * and of load_lora_prefill (lora_gpu.py:165-188).  Bit-exact copy; up to MLORA_SCATTER_MAX_JOBS jobs.
 */
#define MLORA_SCATTER_MAX_JOBS 16
int mlora_pool_scatter(int n_jobs, const void *const *src, void *const *dst_slab, const int32_t *row_elems,
                       const int32_t *pages, int n_slot_pages, int rank, int page_rows, int64_t n_pages,
                       int elt_bytes, void *stream);

/*
 * CPU-assist transport: the GPU side of the path on which host workers compute the LoRA delta while an
 * adapter is still loading (HIP equivalents of the reference's tensor_cp copy family,
 * csrc/cuda_ops.hpp:109-229; no arithmetic here -- the workers are the reference's own processes or any
 * other host code that follows the slot and signal protocol).
 *   mlora_host_alloc / mlora_host_free: pinned host memory mapped into the device address space
 *       (replaces cudaHostRegister of the shared-memory segments, cuda_ops.hpp:109-112); *dev_ptr is the
 *       address kernels use, *host_ptr the one the workers use.  Zero-filled.
 *   mlora_assist_export: hidden [B * tkn, H] (device, 16-bit) -> x_slots [n_slots, slot_tokens, H], request b
 *       at slot b, tokens from row 0; then signals[q][w] = sig_base + sig_stride * q + w for the
 *       B * ceil(tkn / cap) workers of each of the n_proj projections (worker w serves request
 *       w / ceil(tkn / cap), tokens [(w mod ceil(tkn / cap)) * cap, ...)).  One launch for the data, one for
 *       the signals after it.  Replaces Lora_CPU.invoke_lora_async (lora_cpu.py:138-185), codes 2 / 202 / 402.
 *   mlora_assist_import: for projection q, out_slots[q] [n_slots, slot_tokens, H] -> res[q] [B, tkn, out_size],
 *       columns [col0, col0 + out_size) of every row (the rank's share under tensor parallelism).  The
 *       caller launches it once the workers have reset their signals to 0.  Replaces the per-chunk
 *       cudaHtoD2D calls of Lora_CPU.collect_qkv (lora_cpu.py:187-276).
 * x_slots, signals and out_slots are DEVICE addresses of mapped host memory (mlora_host_alloc).
 */
int mlora_host_alloc(int64_t bytes, void **host_ptr, void **dev_ptr);
int mlora_host_free(void *host_ptr);
int mlora_assist_export(const void *hidden, int B, int tkn, int H, void *x_slots, int n_slots, int slot_tokens,
                        int16_t *signals, int n_proj, int n_workers, int cap, int sig_base, int sig_stride,
                        void *stream);
int mlora_assist_import(int n_proj, void *const *res, const void *const *out_slots, int B, int tkn, int H,
                        int out_size, int col0, int n_slots, int slot_tokens, void *stream);

/*
 * Decode (BGMV): for every token t with adapter a = tok_adapter[t] and every projection p
 *     y_p[t] = (accumulate ? y_p[t] : 0) + scaling[a] * (x_p[t] . A_{p,a}) . B_{p,a}
 * shrink and expand fused in one launch, rank-r intermediate kept on chip in fp32.
 * Replaces punica.ops.add_lora_bgmv at lora_gpu.py:138,150,162 plus the
 * `torch.zeros` before it (accumulate = 0) or the `q += q_lora` after it
 * (transformer_layer_infer.py:160-171, accumulate = 1).
 *
 * y, x, a_rows, b_rows, hin, hout are HOST arrays of n_proj entries (device pointers /
 * sizes per projection; projections may share x).  x_p is [T, hin[p]], y_p is [T, hout[p]].
 * The page table, rank and scaling are shared by all projections of the call; n_pages bounds the
 * page ids (rows slab extent) for in-kernel checks.
 * Grouped launch: pass the `work` records written by mlora_pool_gather for this batch with the
 * same `group` (1, 2, 4 or 8; 8 needs max_rank <= 32); tokens of one adapter then share one read
 * of its rows and each workgroup starts from one record instead of walking the tables.
 * With work == NULL every token is its own work item and group must be 1.
 * Two-launch form: with a `workspace` of mlora_bgmv_workspace_bytes(n_proj, T, max hin, max_rank)
 * bytes (and work records) the call runs as a shrink launch and an expand launch over
 * column slices of the items (1024 or 2048 columns, by max_rank), the fp32 intermediate passing through the workspace; on a
 * decode batch with about one item per compute unit this balances the load far better than the
 * fused launch.  workspace == NULL selects the fused launch.  Calls that share a workspace must be
 * ordered on one stream.  Both forms accumulate in fp32 and
 * round once; they differ only in the order the fp32 partial sums of the shrink are added.
 * When the batch makes for many rounds of workgroups (thousands of slices), the two launches cover fewer
 * records than MLORA_WORK_CAP(T): a workgroup serves records b, b + stride, ... of its residue mod 8 and stops
 * at the first empty one.  The layout mlora_pool_gather writes (records in use of each residue first) is what
 * makes that valid; a caller that fills `work` itself must keep it.
 */
int64_t mlora_bgmv_workspace_bytes(int n_proj, int T, int max_hin, int max_rank);
int mlora_bgmv_multi(int n_proj, void *const *y, const void *const *x,
                     const void *const *a_rows, const void *const *b_rows,
                     const int32_t *hin, const int32_t *hout,
                     const int32_t *tok_adapter, int T,
                     const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                     int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                     const int32_t *work, int group,
                     void *workspace, int64_t workspace_bytes,
                     int dtype, int accumulate, void *stream);

/*
 * mlora_bgmv_multi in its two-launch form with no workspace argument and no allocation anywhere on its
 * path.  No counterpart in the reference: it is for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc) and so cannot provide the
 * workspace of the call above.  The fp32 intermediate lives in a file-scope device array of
 * MLORA_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends; a call that
 * needs more (mlora_bgmv_workspace_bytes(n_proj, T, max hin, max_rank): n_proj x T x column slices x rank
 * stride x 4 bytes) returns MLORA_ENOSPACE.  `work` (the records of mlora_pool_gather) is required.  Results
 * are those of mlora_bgmv_multi with a workspace, bit for bit.  The array keeps the previous call's contents;
 * nothing in it has to start at zero (the shrink launch writes every value the expand launch reads).  All
 * calls on one GPU share the one array: calls that overlap on a GPU (two streams, two threads) race; order
 * them on one stream.  The array's device address is looked up on the first call on each device (a runtime
 * query, no allocation): make that first call outside graph capture.
 */
#define MLORA_NOALLOC_SCRATCH_BYTES (16u << 20)
int mlora_bgmv_multi_noalloc(int n_proj, void *const *y, const void *const *x,
                             const void *const *a_rows, const void *const *b_rows,
                             const int32_t *hin, const int32_t *hout,
                             const int32_t *tok_adapter, int T,
                             const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                             int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                             const int32_t *work, int group,
                             int dtype, int accumulate, void *stream);

/* One projection, one token per work item: the plain form of the call above. */
int mlora_bgmv(void *y, const void *x, const void *a_rows, const void *b_rows,
               const int32_t *tok_adapter,
               const int32_t *page_tbl, const int32_t *rank, const float *scaling,
               int T, int hin, int hout, int n_adapters, int max_pages, int page_rows,
               int64_t n_pages, int max_rank,
               int dtype, int accumulate, void *stream);

/*
 * The reference's own layout and call, for drop-in and parity
 * (lora_gpu.py:33-40 pool shapes, :137-138 call):
 *   wa_T_all [N, L, r, hin], wb_T_all [N, L, hout, r] contiguous, indices int64 [T] in [0, N),
 *   y[t] += scale * (x[t] . wa_T_all[idx[t], layer]^T) . wb_T_all[idx[t], layer]^T.
 * An index outside [0, N) leaves that token's row untouched (the reference reads out of
 * bounds there).
 */
int mlora_bgmv_reflayout(void *y, const void *x, const void *wa_T_all, const void *wb_T_all,
                         const int64_t *indices, int T, int N, int L, int r, int hin, int hout,
                         int layer_idx, float scale, int dtype, void *stream);

/*
 * The same call in the grouped two-launch form, for several projections of one layer that use the same index vector
 * (the reference calls add_lora_bgmv three times per layer, for q, k and v: lora_gpu.py:137-138,149-150,161-162).
 *   mlora_reflayout_plan groups the tokens of a batch by adapter once (the plan serves every layer and projection
 *     of the step): indices int64 [T]; plan = device buffer of mlora_reflayout_plan_bytes(T) bytes.  An index outside
 *     [0, N) means "no adapter" for that token.
 *   mlora_bgmv_reflayout_multi: y_p[t] = (accumulate ? y_p[t] : 0) + scale * (x_p[t] . wa_p[idx[t], layer]^T) . wb_p[idx[t], layer]^T
 *     for projection p < n_proj, wa_p [N, L, r, hin_p], wb_p [N, L, hout_p, r] in place (nothing is copied or
 *     transposed); y, x, wa_T_all, wb_T_all, hin, hout are HOST arrays of n_proj entries.  accumulate = 0 writes
 *     zeros for tokens without adapter, so the caller needs no torch.zeros before the call (lora_gpu.py:137).
 *     workspace: mlora_bgmv_workspace_bytes(n_proj, T, max hin, r) bytes; group as given to the plan (1, 2 or 4).
 * Rank 8, 16, 32 or 64 (MLORA_ERANGE otherwise; mlora_bgmv_reflayout takes any rank up to 64).
 */
int64_t mlora_reflayout_plan_bytes(int T);
int mlora_reflayout_plan(const int64_t *indices, int T, int N, int L, int r, int group,
                         void *plan, int64_t plan_bytes, void *stream);
int mlora_bgmv_reflayout_multi(int n_proj, void *const *y, const void *const *x,
                               const void *const *wa_T_all, const void *const *wb_T_all,
                               const int32_t *hin, const int32_t *hout, const void *plan,
                               int T, int N, int L, int r, int layer_idx, float scale, int group,
                               int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Prefill (SGMV): tokens are packed contiguously per segment; segment s covers tokens
 * [seg_start[s], seg_start[s] + seg_len[s]) and uses adapter seg_adapter[s] (negative = none):
 *     y[t] = (accumulate ? y[t] : 0) + scaling[a] * (x[t] . A_a) . B_a
 * computed on MFMA tiles with an fp32 [T, rank] intermediate that stays in `workspace`.
 * Replaces torch.bmm(torch.bmm(x, A), B) at lora_gpu.py:127-128,145-146,157-158 without the
 * per-call weight transposes/copies or the padding to equal prompt length.
 * seg_* are device arrays of n_seg entries.  Segments must not overlap; tokens covered by no
 * segment keep y (accumulate) or get zeros.  workspace: mlora_sgmv_workspace_bytes(T, n_seg).
 */
int64_t mlora_sgmv_workspace_bytes(int T, int n_seg);
int mlora_sgmv(void *y, const void *x, const void *a_rows, const void *b_rows,
               const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
               const int32_t *page_tbl, const int32_t *rank, const float *scaling,
               int T, int hin, int hout, int n_adapters, int max_pages, int page_rows,
               int64_t n_pages, int max_rank,
               int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * The same in two parts, for the usual case in which one batch of segments is applied to many
 * projections and layers: mlora_sgmv_plan writes the tile list and per-tile records (tokens, adapter,
 * rank, scaling, row of every rank row) into the workspace once; mlora_sgmv_planned then runs the
 * arithmetic of one projection against that plan.  The segments, pool tables, T and workspace must be
 * the ones the plan was made with; the plan stays valid until the page table, rank or scaling of a
 * planned adapter changes.  No counterpart in the reference (its prefill re-derives everything per call).
 */
int mlora_sgmv_plan(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                    const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                    int T, int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                    void *workspace, int64_t workspace_bytes, void *stream);
/*
 * mlora_sgmv_plan with the tiles cut at multiples of 64 tokens (and at segment ends) instead of every 64
 * tokens from each segment's start.  Valid for every *_planned call; meant for mlora_gemm_lora_planned, whose
 * 256-row output blocks then meet four tiles (one per 64 rows) except where a segment ends inside a block.
 * No counterpart in the reference.
 */
int mlora_sgmv_plan_aligned(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                            const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                            int T, int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                            void *workspace, int64_t workspace_bytes, void *stream);
int mlora_sgmv_planned(void *y, const void *x, const void *a_rows, const void *b_rows,
                       const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                       const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                       int T, int hin, int hout, int n_adapters, int max_pages, int page_rows,
                       int64_t n_pages, int max_rank,
                       int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Several projections of one layer against one plan, in three launches in all (shrink, reduce, expand)
 * instead of three per projection.  y, x, a_rows, b_rows, hin, hout are HOST arrays of n_proj entries as
 * in mlora_bgmv_multi.  Consecutive projections that are given the same x pointer (q, k, v; gate, up)
 * share its reads in the shrink launch: their workgroups for the same tokens run back to back on one
 * XCD, so x comes from HBM once.  The workspace must hold mlora_sgmv_multi_workspace_bytes(T, n_seg,
 * n_proj) bytes; a plan written by mlora_sgmv_plan into that workspace is valid for any n_proj.
 * Replaces the three torch.bmm pairs of lora_gpu.py:127-128,145-146,157-158 for one layer.
 */
int64_t mlora_sgmv_multi_workspace_bytes(int T, int n_seg, int n_proj);
/*
 * Columns of y that one expand workgroup of such a call covers for a projection of width hout (the library
 * picks 512, or the width whose block count per 64-token tile suits the order its workgroups run in: 640 for
 * hout 5120, 576 for 13824).  Informational, like the workspace sizes; 0 for arguments out of range.  No
 * counterpart in the reference (its prefill is two library GEMMs, lora_gpu.py:127-128).
 */
int mlora_sgmv_expand_cols(int T, int n_seg, int n_proj, int hout);
int mlora_sgmv_multi_planned(int n_proj, void *const *y, const void *const *x,
                             const void *const *a_rows, const void *const *b_rows,
                             const int32_t *hin, const int32_t *hout,
                             const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                             const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                             int T, int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                             int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Base projection and LoRA in one pass, for the projections of one prefill layer:
 *     y[p][t, :] = round16( x[p][t, :] . w[p]  +  scaling[a] * (x[p][t, :] . A_{p,a}) . B_{p,a} ),  a = adapter of t's segment
 * with w[p] the base weight as [hin[p], hout[p]] row-major (the transposed layout lightllm keeps its
 * projection weights in, layer_weights/transformer_layer_weight.py:44-46) and tokens outside every segment,
 * or in a segment without adapter, getting the base product alone.  Replaces torch.mm(x, W) followed by
 * `q += q_lora` (layer_infer/transformer_layer_infer.py:145-147 and :160-171), for which the reference
 * writes y, reads it back and writes it again: here y is written once.  Launches: the SGMV shrink, a scaled
 * reduce, and one GEMM launch for all projections in which the expand rides along as rank / 16 extra MFMA
 * steps per output tile.  The sum is rounded to 16 bits once (the reference rounds the base product, the
 * delta and their sum).  Arrays are HOST arrays of n_proj entries as in mlora_sgmv_multi_planned; the
 * workspace must hold mlora_sgmv_multi_workspace_bytes(T, n_seg, n_proj) bytes and a plan written by
 * mlora_sgmv_plan for these segments.  n_seg = 0 runs the base products alone (workspace and pool may be
 * NULL).  Limits: every w[p] and every B rows slab smaller than 4 GiB.
 */
int mlora_gemm_lora_planned(int n_proj, void *const *y, const void *const *x, const void *const *w,
                            const void *const *a_rows, const void *const *b_rows,
                            const int32_t *hin, const int32_t *hout,
                            const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                            const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                            int T, int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                            int dtype, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * The reference's prefill call on its own layout (lora_gpu.py:125-128): request b uses
 * adapter slot b; x [B, Lpad, hin]; A_T [>=B, L, r, hin]; B_T [>=B, L, hout, r];
 * y [B, Lpad, hout] = (x[b] . A_T[b, layer]^T) . B_T[b, layer]^T   (y is overwritten).
 */
int mlora_prefill_reflayout(void *y, const void *x, const void *A_T, const void *B_T,
                            int B, int Lpad, int L, int r, int hin, int hout, int layer_idx,
                            int dtype, void *workspace, int64_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_H */
