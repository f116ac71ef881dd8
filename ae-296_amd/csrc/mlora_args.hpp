// Kernel argument blocks and launcher prototypes shared between the kernels and
// the C ABI layer.  Plain structs passed by value in the kernarg segment.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlora {

constexpr int MAX_PROJ = 8;
constexpr int MAX_RANK = 64;
// Decode work record (int32 words): [0] tokens in the item (0 = empty), [1] adapter (-1 = none),
// [2] rank, [3] scaling (float bits), [4..11] token ids, [12..15] zero, [16..79] row of rank row j (-1 = absent).
constexpr int WORK_WORDS = 80;
constexpr int WORK_ROWS_AT = 16;
// Prefill tile record (int32 words): [0] tokens in the tile (0 = nothing to do), [1] adapter (-1 = none),
// [2] rank, [3] scaling (float bits), [4] first token, [5] segment, [6..15] zero, [16..79] row of rank row j.
constexpr int TILE_WORDS = 80;
constexpr int TILE_ROWS_AT = 16;

// How the rank rows of an adapter are found inside a rows slab.
struct PoolView {
    const int32_t *a_tbl;      // [n_adapters, max_pages] or nullptr (dense)
    const int32_t *b_tbl;
    const int32_t *rank;       // [n_adapters] or nullptr (uniform_rank)
    const float *scaling;      // [n_adapters] or nullptr (uniform_scale)
    int n_adapters;
    int max_pages;
    int page_shift;            // log2(page_rows)
    int uniform_rank;
    float uniform_scale;
    long long n_rows_a;        // slab extents in rows, for in-kernel bounds checks
    long long n_rows_b;
    long long a_dense_stride;  // rows between adapters when a_tbl == nullptr
    long long b_dense_stride;  // rows (B as rank rows) or elements (B^T blocks) when b_tbl == nullptr
};

struct BgmvArgs {
    void *y[MAX_PROJ];
    const void *x[MAX_PROJ];
    const void *a_rows[MAX_PROJ];
    const void *b_rows[MAX_PROJ];
    int hin[MAX_PROJ];
    int hout[MAX_PROJ];
    PoolView pool;
    const int32_t *tok_adapter;    // [T] int32, or nullptr when tok_adapter64 is used
    const int64_t *tok_adapter64;  // [T] int64 (reference layout call)
    const int32_t *work;           // work records in launch order (nullptr => one token per workgroup)
    int work_cap;                  // records the gather wrote (in use or empty), a multiple of 8
    int items_cap;                 // records that can be in use for this T, group and pool (<= work_cap, multiple of 8)
    int T;
    int n_proj;
    int accumulate;
    int b_transposed;              // two-launch form on the reference layout: b_rows[p] is [n_adapters, ref_layers, hout, rank] (this layer's
    int ref_layers;                //   block first), adapter a's [hout, rank] block starts a * ref_layers * hout * rank elements in
    float *vws;                    // two-launch form: partial sums [n_proj, T, ks_max, rank stride] (else nullptr)
    int ks_max;                    // shrink slices of the widest hin (stride of the partial sums)
    int cs_max;                    // expand slices of the widest hout
    // two-launch form: the (projection, slice) pairs that exist, numbered consecutively; sh_end[p] / ex_end[p] is
    // the number of shrink / expand slices of projections 0..p
    int sh_end[MAX_PROJ];
    int ex_end[MAX_PROJ];
    // two-launch form: records the shrink / expand grid covers; a workgroup walks records b, b + stride, ... < items_cap
    // (set by the launcher)
    int rec_stride_sh, rec_stride_ex;
};

constexpr int SCATTER_MAX_JOBS = 16;
struct ScatterArgs {
    const void *src[SCATTER_MAX_JOBS];   // [rank, row_bytes] contiguous rank rows
    void *dst[SCATTER_MAX_JOBS];         // rows slab base
    int row_bytes[SCATTER_MAX_JOBS];     // multiple of 16
    int pages[64];                       // page id of rank rows [k * page_rows, (k + 1) * page_rows)
    int n_jobs, rank, page_shift;
    long long n_pages;
};

constexpr int ASSIST_MAX_PROJ = 4;
struct AssistArgs {
    const void *dev;                       // export: hidden states [B * tkn, H] (device)
    void *host_slots[ASSIST_MAX_PROJ];     // export: [0] = request slots; import: result slots per projection (mapped host)
    void *dev_out[ASSIST_MAX_PROJ];        // import: [B, tkn, out] per projection (device)
    int16_t *signals;                      // [n_proj, n_workers] (mapped host)
    int B, tkn, H, out, col0;
    int n_slots, slot_tokens;
    int n_proj, n_workers, n_active;
    int sig_base, sig_stride;
};

struct GatherArgs {
    const int32_t *tok_adapter;    // [T] int32, or nullptr when tok_adapter64 is used
    const int64_t *tok_adapter64;  // [T] int64 (the reference's index vector); an id outside [0, n_adapters) means no adapter
    const int32_t *page_tbl;       // nullptr: dense pool, rank row j of adapter a is row a * dense_stride + j
    const int32_t *rank;           // nullptr: every adapter has uniform_rank
    const float *scaling;          // nullptr: every adapter has uniform_scale
    long long dense_stride;
    long long n_rows_dense;        // rows a dense slab holds (bounds the recorded rows)
    int uniform_rank;
    float uniform_scale;
    int T, n_adapters, max_pages, page_rows, group;
    long long n_pages;             // pages in a rows slab (bounds the recorded rows)
    int32_t *work;                 // [work_cap * WORK_WORDS] decode work records, or nullptr
    int work_cap;
    int32_t *out_row_off;
    int32_t *out_rank;
    float *out_scale;
    int32_t *perm, *seg_start, *seg_len, *seg_adapter;
    int32_t *chunk_start, *chunk_len, *chunk_adapter;
    int32_t *counters;
};

// Whether a projection with `ncb` column blocks per tile runs its expand workgroups tile-major (the blocks of a
// tile numbered up to the next multiple of eight): only when at most an eighth of the numbers stays unused.
__host__ __device__ inline bool tile_major(int ncb) { return (((ncb + 7) & ~7) - ncb) * 8 <= ncb; }

// One projection of a prefill call.
struct SgmvProj {
    void *y;
    const void *x;
    const void *a_rows;
    const void *b_rows;
    float *v;              // [ksplit, T, MAX_RANK] fp32 partial intermediates
    uint16_t *vhi;         // [T, MAX_RANK] 16-bit hi part of the summed intermediate
    uint16_t *vlo;         // [T, MAX_RANK] 16-bit lo part
    int hin, hout;
    int ksplit;            // K splits of the shrink
    int cols, ncb;         // expand: columns per workgroup, column blocks
};

struct SgmvArgs {
    SgmvProj pr[MAX_PROJ];
    int n_proj;
    // Shrink launch: up to three consecutive projections that read the same x form a group, served by one
    // workgroup per (tile, K split): x comes from HBM once per group and is multiplied with every member's A.
    // grp_end[g] = first workgroup id after group g.
    int n_grp;
    int grp_first[MAX_PROJ], grp_n[MAX_PROJ];
    unsigned grp_end[MAX_PROJ];
    unsigned ex_end[MAX_PROJ];     // expand launch: first workgroup id after projection p
    PoolView pool;
    const int32_t *seg_start;
    const int32_t *seg_len;
    const int32_t *seg_adapter;
    int n_seg;
    int T;
    int accumulate;
    int b_transposed;      // B given as [hout, r] blocks (reference layout)
    int seg_uniform_len;   // > 0: segment s covers [s*len, (s+1)*len), adapter s (reference prefill)
    int tile_aligned;      // plan: cut tiles at multiples of 64 tokens (and at segment ends) instead of every 64 tokens of a segment
    // workspace carve-up
    int32_t *tile_seg;     // [max_tiles]
    int32_t *tile_tok0;
    int32_t *tile_ntok;
    int32_t *n_tiles;      // [1]
    int32_t *tok_cover;    // [T] 1 where a token belongs to a tile (written by the plan): rows of y = delta mode outside are zeroed
    int32_t *tile_rec;     // [max_tiles * TILE_WORDS] per-tile records (layout below)
    int max_tiles;
};

// One projection of a base GEMM + LoRA call.
struct GemmProj {
    void *y;               // [T, hout], written once
    const void *x;         // [T, hin]
    const void *w;         // [hin, hout] row-major base weight
    const void *b_rows;    // B rows slab of the pool
    const float *v;        // [ksplit, T, MAX_RANK] shrink partials (read by the scaled reduce)
    uint16_t *vhi;         // [T, MAX_RANK] hi part of scaling * intermediate
    uint16_t *vlo;         // [T, MAX_RANK] lo part
    int hin, hout;
    int ksplit;
    int ntn;               // column tiles (set by the launcher)
    unsigned end;          // first workgroup id after this projection (set by the launcher)
};

struct GemmLoraArgs {
    GemmProj pr[MAX_PROJ];
    int n_proj;
    int T;
    int ntm;               // row tiles (set by the launcher)
    int lora;              // 0: base product only
    int rmax;              // rank columns the intermediate holds (16, 32 or 64; set by the launcher)
    const int32_t *tile_rec;   // prefill plan records
    const int32_t *n_tiles;    // [1]
    int max_tiles;
    long long n_rows_b;
};

// launchers (defined next to their kernels); return hipError_t as int
int launch_bgmv(const BgmvArgs &a, int dtype, int group, int max_rank, bool b_transposed, hipStream_t s);
int launch_bgmv_split(const BgmvArgs &a, int dtype, int group, int max_rank, hipStream_t s);   // a.b_transposed: max_rank is the pool's rank (8, 16, 32 or 64)
int bgmv_split_rank_stride(int max_rank);
void bgmv_split_slices(int max_rank, int *shrink_chunks, int *expand_chunks, bool transposed_b = false);   // slice widths in 16-byte chunks
int launch_gather(const GatherArgs &a, hipStream_t s);
int launch_scatter(const ScatterArgs &a, hipStream_t s);
int launch_assist_export(const AssistArgs &a, hipStream_t s);
int launch_assist_import(const AssistArgs &a, hipStream_t s);
constexpr int SGMV_PLAN = 1;    // write the tile list and records into the workspace
constexpr int SGMV_APPLY = 2;   // shrink, reduce, expand (the workspace already holds the plan unless SGMV_PLAN is set too)
constexpr int SGMV_SHRINK = 4;  // the shrink launch alone: its partial sums feed the base GEMM + LoRA kernel
int launch_sgmv(const SgmvArgs &a, int dtype, int max_rank, int phases, hipStream_t s);
int launch_gemm_lora(const GemmLoraArgs &a, int dtype, int max_rank, hipStream_t s);
// compute units of the current device (asked once per device; 256 when the query fails)
int device_compute_units();

}  // namespace mlora
