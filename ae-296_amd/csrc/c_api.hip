// extern "C" surface of libmlora_hip.so (declared in include/mlora.h): argument
// validation on the host, then one or two kernel launches on the caller's stream.
// No allocation, no synchronisation, no state kept between calls.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/mlora.h"
#include "mlora_args.hpp"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int log2_exact(int v)
{
    for (int s = 0; s < 31; s++)
        if ((1 << s) == v) return s;
    return -1;
}

int check_pool(mlora::PoolView &pv, const int32_t *page_tbl, const int32_t *rank, const float *scaling,
               int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank)
{
    const int32_t *a_tbl = page_tbl, *b_tbl = page_tbl;
    const int64_t n_pages_a = n_pages, n_pages_b = n_pages;
    if (!page_tbl || !rank || !scaling) return fail(MLORA_EINVAL, "page table, rank and scaling must not be NULL");
    if (n_adapters <= 0) return fail(MLORA_EINVAL, "n_adapters must be positive (got %d)", n_adapters);
    const int shift = log2_exact(page_rows);
    if (shift < 0 || page_rows > 64) return fail(MLORA_EINVAL, "page_rows must be a power of two in 1..64 (got %d)", page_rows);
    if (max_pages <= 0) return fail(MLORA_EINVAL, "max_pages must be positive (got %d)", max_pages);
    if (max_rank < 1 || max_rank > MLORA_MAX_RANK) return fail(MLORA_ERANGE, "max_rank must be in 1..%d (got %d)", MLORA_MAX_RANK, max_rank);
    if ((int64_t)max_pages * page_rows < max_rank)
        return fail(MLORA_ERANGE, "max_pages * page_rows = %lld cannot hold max_rank %d", (long long)max_pages * page_rows, max_rank);
    if (n_pages <= 0) return fail(MLORA_EINVAL, "n_pages must be positive");
    if (n_pages_a * page_rows > 0x7fffffffLL || n_pages_b * page_rows > 0x7fffffffLL)
        return fail(MLORA_ERANGE, "a rows slab may hold at most 2^31-1 rows");
    pv.a_tbl = a_tbl; pv.b_tbl = b_tbl; pv.rank = rank; pv.scaling = scaling;
    pv.n_adapters = n_adapters; pv.max_pages = max_pages; pv.page_shift = shift;
    pv.uniform_rank = 0; pv.uniform_scale = 0.f;
    pv.n_rows_a = n_pages_a * page_rows; pv.n_rows_b = n_pages_b * page_rows;
    pv.a_dense_stride = 0; pv.b_dense_stride = 0;
    return MLORA_OK;
}

// Device memory for mlora_bgmv_multi_noalloc: the fp32 intermediate of the two-launch decode form, for
// callers that cannot allocate.  Every GPU the library runs on holds its own copy of the array at its own
// address until the process ends; host code only ever uses the per-device address looked up below, never
// the array's name (which on the host is a stand-in, not a device address).
constexpr size_t SCRATCH_BYTES = MLORA_NOALLOC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

constexpr int SCRATCH_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};

// Address of the current device's copy of `scratch` (looked up once per device); nullptr + error text on failure.
void *scratch_of_current_device()
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { fail(MLORA_ELAUNCH, "hipGetDevice failed: %s", hipGetErrorString(e)); return nullptr; }
    if (dev < 0 || dev >= SCRATCH_MAX_DEVICES) { fail(MLORA_ERANGE, "device ordinal %d outside [0, %d)", dev, SCRATCH_MAX_DEVICES); return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            fail(MLORA_ELAUNCH, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

int check_dims(int hin, int hout)
{
    if (hin <= 0 || hout <= 0) return fail(MLORA_EINVAL, "hin and hout must be positive (got %d, %d)", hin, hout);
    if ((hin & 7) || (hout & 7)) return fail(MLORA_EALIGN, "hin and hout must be multiples of 8 (got %d, %d)", hin, hout);
    return MLORA_OK;
}

}  // namespace

namespace mlora {

int device_compute_units()
{
    static std::mutex mu;
    static int cus[SCRATCH_MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_MAX_DEVICES) return 256;
    std::lock_guard<std::mutex> lock(mu);
    if (!cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    return cus[dev];
}

}  // namespace mlora

extern "C" {

const char *mlora_last_error(void) { return g_err; }
int mlora_version(void) { return 100; }

int mlora_pool_gather(const int32_t *tok_adapter, int T, const int32_t *page_tbl, const int32_t *rank,
                      const float *scaling, int n_adapters, int max_pages, int page_rows, int64_t n_pages,
                      int32_t *out_row_off, int32_t *out_rank, float *out_scale, int32_t *perm,
                      int32_t *seg_start, int32_t *seg_len, int32_t *seg_adapter, int32_t *chunk_start,
                      int32_t *chunk_len, int32_t *chunk_adapter, int group, int32_t *counters, int32_t *work,
                      void *stream)
{
    if (T < 0) return fail(MLORA_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_OK;
    if (!tok_adapter) return fail(MLORA_EINVAL, "tok_adapter must not be NULL");
    if (n_adapters <= 0 || n_adapters > (1 << 18)) return fail(MLORA_ERANGE, "n_adapters must be in 1..262144 (got %d)", n_adapters);
    const bool per_tok = out_row_off || out_rank || out_scale;
    if (per_tok) {
        if (!page_tbl || !rank || !scaling) return fail(MLORA_EINVAL, "page_tbl, rank and scaling are needed for the per-token view");
        if (max_pages <= 0 || page_rows <= 0) return fail(MLORA_EINVAL, "max_pages and page_rows must be positive");
    }
    const bool grouped = perm || seg_start || seg_len || seg_adapter || chunk_start || chunk_len || chunk_adapter || counters || work;
    if (grouped) {
        if (!(perm && seg_start && seg_len && seg_adapter && chunk_start && chunk_len && chunk_adapter && counters))
            return fail(MLORA_EINVAL, "the grouped view needs all of perm, seg_*, chunk_* and counters");
        if (T > MLORA_GATHER_MAX_T) return fail(MLORA_ERANGE, "T = %d exceeds MLORA_GATHER_MAX_T = %d", T, MLORA_GATHER_MAX_T);
        if (group != 1 && group != 2 && group != 4 && group != 8) return fail(MLORA_EINVAL, "group must be 1, 2, 4 or 8 (got %d)", group);
        if (work) {
            if (!page_tbl || !rank || !scaling) return fail(MLORA_EINVAL, "page_tbl, rank and scaling are needed for the work records");
            if (max_pages <= 0 || page_rows <= 0 || n_pages <= 0) return fail(MLORA_EINVAL, "max_pages, page_rows and n_pages must be positive");
            if (n_pages * (int64_t)page_rows > 0x7fffffffLL) return fail(MLORA_ERANGE, "a rows slab may hold at most 2^31-1 rows");
        }
    }
    if (!per_tok && !grouped) return MLORA_OK;
    mlora::GatherArgs a;
    memset(&a, 0, sizeof(a));
    a.tok_adapter = tok_adapter; a.page_tbl = page_tbl; a.rank = rank; a.scaling = scaling;
    a.T = T; a.n_adapters = n_adapters; a.max_pages = max_pages > 0 ? max_pages : 1;
    a.page_rows = page_rows > 0 ? page_rows : 1; a.group = grouped ? group : 1;
    a.out_row_off = out_row_off; a.out_rank = out_rank; a.out_scale = out_scale;
    a.perm = perm; a.seg_start = seg_start; a.seg_len = seg_len; a.seg_adapter = seg_adapter;
    a.chunk_start = chunk_start; a.chunk_len = chunk_len; a.chunk_adapter = chunk_adapter; a.counters = counters;
    a.n_pages = n_pages; a.work = work; a.work_cap = MLORA_WORK_CAP(T);
    const int rc = mlora::launch_gather(a, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "gather launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_pool_scatter(int n_jobs, const void *const *src, void *const *dst_slab, const int32_t *row_elems,
                       const int32_t *pages, int n_slot_pages, int rank, int page_rows, int64_t n_pages,
                       int elt_bytes, void *stream)
{
    if (n_jobs < 0 || n_jobs > MLORA_SCATTER_MAX_JOBS) return fail(MLORA_ERANGE, "n_jobs must be in 0..%d (got %d)", MLORA_SCATTER_MAX_JOBS, n_jobs);
    if (n_jobs == 0) return MLORA_OK;
    if (!src || !dst_slab || !row_elems || !pages) return fail(MLORA_EINVAL, "NULL argument array");
    if (rank < 1 || rank > MLORA_MAX_RANK) return fail(MLORA_ERANGE, "rank must be in 1..%d (got %d)", MLORA_MAX_RANK, rank);
    if (page_rows < 1 || page_rows > 64 || (page_rows & (page_rows - 1))) return fail(MLORA_EINVAL, "page_rows must be a power of two in 1..64 (got %d)", page_rows);
    if (elt_bytes != 1 && elt_bytes != 2 && elt_bytes != 4) return fail(MLORA_EINVAL, "elt_bytes must be 1, 2 or 4 (got %d)", elt_bytes);
    if (n_pages <= 0 || n_pages * (int64_t)page_rows > 0x7fffffffLL) return fail(MLORA_ERANGE, "n_pages out of range");
    const int need = (rank + page_rows - 1) / page_rows;
    if (n_slot_pages < need) return fail(MLORA_ERANGE, "rank %d needs %d pages, %d given", rank, need, n_slot_pages);
    mlora::ScatterArgs a;
    memset(&a, 0, sizeof(a));
    for (int k = 0; k < 64; k++) a.pages[k] = -1;
    for (int k = 0; k < need; k++) {
        if (pages[k] < 0 || pages[k] >= n_pages) return fail(MLORA_ERANGE, "page id %d outside [0, %lld)", pages[k], (long long)n_pages);
        a.pages[k] = pages[k];
    }
    for (int j = 0; j < n_jobs; j++) {
        if (!src[j] || !dst_slab[j]) return fail(MLORA_EINVAL, "job %d: NULL device pointer", j);
        const int64_t rb = (int64_t)row_elems[j] * elt_bytes;
        if (row_elems[j] <= 0 || (rb & 15) || rb > 0x7fffffffLL) return fail(MLORA_EALIGN, "job %d: a row must be a positive multiple of 16 bytes", j);
        if (!aligned16(src[j]) || !aligned16(dst_slab[j])) return fail(MLORA_EALIGN, "job %d: device pointers must be 16-byte aligned", j);
        a.src[j] = src[j]; a.dst[j] = dst_slab[j]; a.row_bytes[j] = (int)rb;
    }
    a.n_jobs = n_jobs; a.rank = rank; a.n_pages = n_pages;
    a.page_shift = 0;
    while ((1 << a.page_shift) < page_rows) a.page_shift++;
    const int rc = mlora::launch_scatter(a, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "scatter launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_host_alloc(int64_t bytes, void **host_ptr, void **dev_ptr)
{
    if (bytes <= 0 || !host_ptr || !dev_ptr) return fail(MLORA_EINVAL, "bytes must be positive and the out pointers non-NULL");
    void *h = nullptr, *d = nullptr;
    hipError_t e = hipHostMalloc(&h, (size_t)bytes, hipHostMallocMapped | hipHostMallocPortable);
    if (e != hipSuccess) return fail(MLORA_ELAUNCH, "hipHostMalloc of %lld bytes failed: %s", (long long)bytes, hipGetErrorString(e));
    e = hipHostGetDevicePointer(&d, h, 0);
    if (e != hipSuccess) { (void)hipHostFree(h); return fail(MLORA_ELAUNCH, "hipHostGetDevicePointer failed: %s", hipGetErrorString(e)); }
    memset(h, 0, (size_t)bytes);
    *host_ptr = h; *dev_ptr = d;
    return MLORA_OK;
}

int mlora_host_free(void *host_ptr)
{
    if (!host_ptr) return MLORA_OK;
    const hipError_t e = hipHostFree(host_ptr);
    if (e != hipSuccess) return fail(MLORA_ELAUNCH, "hipHostFree failed: %s", hipGetErrorString(e));
    return MLORA_OK;
}

static int assist_dims(int B, int tkn, int H, int n_slots, int slot_tokens)
{
    if (B < 0 || tkn < 0) return fail(MLORA_EINVAL, "B and tkn must be >= 0 (got %d, %d)", B, tkn);
    if (H <= 0 || (H & 7)) return fail(MLORA_EALIGN, "H must be a positive multiple of 8 (got %d)", H);
    if (n_slots <= 0 || slot_tokens <= 0) return fail(MLORA_EINVAL, "n_slots and slot_tokens must be positive");
    if (B > n_slots) return fail(MLORA_ERANGE, "%d requests do not fit %d request slots", B, n_slots);
    if (tkn > slot_tokens) return fail(MLORA_ERANGE, "%d tokens per request do not fit a slot of %d", tkn, slot_tokens);
    return MLORA_OK;
}

int mlora_assist_export(const void *hidden, int B, int tkn, int H, void *x_slots, int n_slots, int slot_tokens,
                        int16_t *signals, int n_proj, int n_workers, int cap, int sig_base, int sig_stride, void *stream)
{
    int rc = assist_dims(B, tkn, H, n_slots, slot_tokens);
    if (rc) return rc;
    if (B == 0 || tkn == 0) return MLORA_OK;
    if (!hidden || !x_slots || !signals) return fail(MLORA_EINVAL, "NULL pointer");
    if (!aligned16(hidden) || !aligned16(x_slots)) return fail(MLORA_EALIGN, "hidden and x_slots must be 16-byte aligned");
    if (n_proj < 1 || n_proj > mlora::ASSIST_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", mlora::ASSIST_MAX_PROJ, n_proj);
    if (cap <= 0) return fail(MLORA_EINVAL, "cap (tokens per worker) must be positive");
    const int64_t active = (int64_t)B * ((tkn - 1) / cap + 1);      // one worker per (request, chunk of <= cap tokens)
    if (active > n_workers) return fail(MLORA_ERANGE, "%lld workers needed per projection, %d available", (long long)active, n_workers);
    if (sig_base < 2 || sig_stride < active || (int64_t)sig_base + (int64_t)sig_stride * n_proj > 32767)
        return fail(MLORA_ERANGE, "signal codes must be > 1, distinct per projection and fit 16 bits");
    mlora::AssistArgs a;
    memset(&a, 0, sizeof(a));
    a.dev = hidden; a.host_slots[0] = x_slots; a.signals = signals;
    a.B = B; a.tkn = tkn; a.H = H; a.n_slots = n_slots; a.slot_tokens = slot_tokens;
    a.n_proj = n_proj; a.n_workers = n_workers; a.n_active = (int)active; a.sig_base = sig_base; a.sig_stride = sig_stride;
    rc = mlora::launch_assist_export(a, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "export launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_assist_import(int n_proj, void *const *res, const void *const *out_slots, int B, int tkn, int H, int out_size,
                        int col0, int n_slots, int slot_tokens, void *stream)
{
    int rc = assist_dims(B, tkn, H, n_slots, slot_tokens);
    if (rc) return rc;
    if (B == 0 || tkn == 0) return MLORA_OK;
    if (n_proj < 1 || n_proj > mlora::ASSIST_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", mlora::ASSIST_MAX_PROJ, n_proj);
    if (!res || !out_slots) return fail(MLORA_EINVAL, "NULL argument array");
    if (out_size <= 0 || (out_size & 7) || col0 < 0 || (col0 & 7) || col0 + out_size > H)
        return fail(MLORA_EALIGN, "out_size and col0 must be multiples of 8 with col0 + out_size <= H");
    mlora::AssistArgs a;
    memset(&a, 0, sizeof(a));
    for (int q = 0; q < n_proj; q++) {
        if (!res[q] || !out_slots[q]) return fail(MLORA_EINVAL, "projection %d: NULL pointer", q);
        if (!aligned16(res[q]) || !aligned16(out_slots[q])) return fail(MLORA_EALIGN, "projection %d: pointers must be 16-byte aligned", q);
        a.dev_out[q] = res[q]; a.host_slots[q] = const_cast<void *>(out_slots[q]);
    }
    a.B = B; a.tkn = tkn; a.H = H; a.out = out_size; a.col0 = col0; a.n_slots = n_slots; a.slot_tokens = slot_tokens;
    a.n_proj = n_proj;
    rc = mlora::launch_assist_import(a, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "import launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int64_t mlora_bgmv_workspace_bytes(int n_proj, int T, int max_hin, int max_rank)
{
    if (n_proj < 1 || T < 1 || max_hin < 1) return 0;
    int ksc, nte;
    mlora::bgmv_split_slices(max_rank, &ksc, &nte);
    const int64_t ks = (max_hin + ksc * 8 - 1) / (ksc * 8);
    return (int64_t)n_proj * T * ks * mlora::bgmv_split_rank_stride(max_rank) * (int64_t)sizeof(float);
}

// use_scratch: the two-launch form with the library's own per-device scratch array as its workspace
static int bgmv_multi_impl(int n_proj, void *const *y, const void *const *x, const void *const *a_rows,
                     const void *const *b_rows, const int32_t *hin, const int32_t *hout,
                     const int32_t *tok_adapter, int T, const int32_t *page_tbl, const int32_t *rank,
                     const float *scaling, int n_adapters, int max_pages, int page_rows, int64_t n_pages,
                     int max_rank, const int32_t *work, int group, void *workspace, int64_t workspace_bytes,
                     bool use_scratch, int dtype, int accumulate, void *stream)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (n_proj < 1 || n_proj > MLORA_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", MLORA_MAX_PROJ, n_proj);
    if (T < 0) return fail(MLORA_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_OK;
    if (!y || !x || !a_rows || !b_rows || !hin || !hout) return fail(MLORA_EINVAL, "per-projection arrays must not be NULL");
    if (!tok_adapter) return fail(MLORA_EINVAL, "tok_adapter must not be NULL");
    mlora::BgmvArgs a;
    memset(&a, 0, sizeof(a));
    int rc = check_pool(a.pool, page_tbl, rank, scaling, n_adapters, max_pages, page_rows, n_pages, max_rank);
    if (rc) return rc;
    if (work) {
        if (group != 1 && group != 2 && group != 4 && group != 8) return fail(MLORA_EINVAL, "group must be 1, 2, 4 or 8 (got %d)", group);
        if (group == 8 && max_rank > 32) return fail(MLORA_ERANGE, "group 8 supports max_rank <= 32 (got %d); use group 4", max_rank);
        if (!aligned16(work)) return fail(MLORA_EALIGN, "work records must be 16-byte aligned");
    } else if (group != 1) {
        return fail(MLORA_EINVAL, "group must be 1 when work is NULL (got %d)", group);
    }
    if ((workspace || use_scratch) && !work) return fail(MLORA_EINVAL, "the two-launch form needs the work records");
    int max_hin = 0, max_hout = 0;
    for (int p = 0; p < n_proj; p++) {
        if (!y[p] || !x[p] || !a_rows[p] || !b_rows[p]) return fail(MLORA_EINVAL, "projection %d: NULL device pointer", p);
        if (!aligned16(y[p]) || !aligned16(x[p]) || !aligned16(a_rows[p]) || !aligned16(b_rows[p]))
            return fail(MLORA_EALIGN, "projection %d: device pointers must be 16-byte aligned", p);
        rc = check_dims(hin[p], hout[p]);
        if (rc) return rc;
        a.y[p] = y[p]; a.x[p] = x[p]; a.a_rows[p] = a_rows[p]; a.b_rows[p] = b_rows[p];
        a.hin[p] = hin[p]; a.hout[p] = hout[p];
        max_hin = hin[p] > max_hin ? hin[p] : max_hin;
        max_hout = hout[p] > max_hout ? hout[p] : max_hout;
    }
    a.tok_adapter = tok_adapter; a.tok_adapter64 = nullptr;
    a.work = work; a.work_cap = MLORA_WORK_CAP(T);
    {
        // Work items in use <= T/group + segments + 1 (one short piece per adapter present, one for the
        // adapter-less tokens); the gather packs them into the first records, so the rest needs no workgroup.
        const int g = group > 0 ? group : 1;
        const int64_t segs = T < n_adapters ? T : n_adapters;
        const int64_t bound = ((int64_t)(T + g - 1) / g + segs + 1 + 7) / 8 * 8;
        a.items_cap = bound < a.work_cap ? (int)bound : a.work_cap;
    }
    a.T = T; a.n_proj = n_proj; a.accumulate = accumulate ? 1 : 0;
    if (use_scratch) {
        const int64_t need = mlora_bgmv_workspace_bytes(n_proj, T, max_hin, max_rank);
        if (need > (int64_t)SCRATCH_BYTES)
            return fail(MLORA_ENOSPACE, "this call needs %lld bytes of intermediate, the allocation-free entry point holds %lld "
                        "(n_proj x T x column slices x rank); use mlora_bgmv_multi with a workspace", (long long)need, (long long)SCRATCH_BYTES);
        workspace = scratch_of_current_device();
        if (!workspace) return MLORA_ELAUNCH;
        workspace_bytes = (int64_t)SCRATCH_BYTES;
    }
    if (workspace) {
        const int64_t need = mlora_bgmv_workspace_bytes(n_proj, T, max_hin, max_rank);
        if (workspace_bytes < need)
            return fail(MLORA_ENOSPACE, "workspace holds %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
        if (!aligned16(workspace)) return fail(MLORA_EALIGN, "workspace must be 16-byte aligned");
        a.vws = static_cast<float *>(workspace);
        int ksc, nte;
        mlora::bgmv_split_slices(max_rank, &ksc, &nte);
        a.ks_max = (max_hin + ksc * 8 - 1) / (ksc * 8);
        a.cs_max = (max_hout + nte * 8 - 1) / (nte * 8);
        int sh = 0, ex = 0;
        for (int p = 0; p < n_proj; p++) {
            sh += (hin[p] + ksc * 8 - 1) / (ksc * 8);
            ex += (hout[p] + nte * 8 - 1) / (nte * 8);
            a.sh_end[p] = sh; a.ex_end[p] = ex;
        }
        rc = mlora::launch_bgmv_split(a, dtype, group, max_rank, static_cast<hipStream_t>(stream));
    } else {
        rc = mlora::launch_bgmv(a, dtype, group, max_rank, false, static_cast<hipStream_t>(stream));
    }
    if (rc) return fail(MLORA_ELAUNCH, "bgmv launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_bgmv_multi(int n_proj, void *const *y, const void *const *x, const void *const *a_rows,
                     const void *const *b_rows, const int32_t *hin, const int32_t *hout,
                     const int32_t *tok_adapter, int T, const int32_t *page_tbl, const int32_t *rank,
                     const float *scaling, int n_adapters, int max_pages, int page_rows, int64_t n_pages,
                     int max_rank, const int32_t *work, int group, void *workspace, int64_t workspace_bytes,
                     int dtype, int accumulate, void *stream)
{
    return bgmv_multi_impl(n_proj, y, x, a_rows, b_rows, hin, hout, tok_adapter, T, page_tbl, rank, scaling, n_adapters,
                           max_pages, page_rows, n_pages, max_rank, work, group, workspace, workspace_bytes, false,
                           dtype, accumulate, stream);
}

int mlora_bgmv_multi_noalloc(int n_proj, void *const *y, const void *const *x, const void *const *a_rows,
                             const void *const *b_rows, const int32_t *hin, const int32_t *hout,
                             const int32_t *tok_adapter, int T, const int32_t *page_tbl, const int32_t *rank,
                             const float *scaling, int n_adapters, int max_pages, int page_rows, int64_t n_pages,
                             int max_rank, const int32_t *work, int group, int dtype, int accumulate, void *stream)
{
    if (!work) return fail(MLORA_EINVAL, "mlora_bgmv_multi_noalloc needs the work records of mlora_pool_gather");
    return bgmv_multi_impl(n_proj, y, x, a_rows, b_rows, hin, hout, tok_adapter, T, page_tbl, rank, scaling, n_adapters,
                           max_pages, page_rows, n_pages, max_rank, work, group, nullptr, 0, true,
                           dtype, accumulate, stream);
}

int mlora_bgmv(void *y, const void *x, const void *a_rows, const void *b_rows, const int32_t *tok_adapter,
               const int32_t *page_tbl, const int32_t *rank, const float *scaling, int T, int hin, int hout,
               int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank, int dtype,
               int accumulate, void *stream)
{
    void *ys[1] = {y};
    const void *xs[1] = {x}, *as[1] = {a_rows}, *bs[1] = {b_rows};
    const int32_t hi[1] = {hin}, ho[1] = {hout};
    return mlora_bgmv_multi(1, ys, xs, as, bs, hi, ho, tok_adapter, T, page_tbl, rank, scaling, n_adapters,
                            max_pages, page_rows, n_pages, max_rank, nullptr, 1, nullptr, 0, dtype, accumulate, stream);
}

int mlora_bgmv_reflayout(void *y, const void *x, const void *wa_T_all, const void *wb_T_all,
                         const int64_t *indices, int T, int N, int L, int r, int hin, int hout, int layer_idx,
                         float scale, int dtype, void *stream)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (T < 0) return fail(MLORA_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_OK;
    if (!y || !x || !wa_T_all || !wb_T_all || !indices) return fail(MLORA_EINVAL, "NULL device pointer");
    if (N <= 0 || L <= 0) return fail(MLORA_EINVAL, "N and L must be positive (got %d, %d)", N, L);
    if (layer_idx < 0 || layer_idx >= L) return fail(MLORA_ERANGE, "layer_idx %d outside [0, %d)", layer_idx, L);
    if (r < 1 || r > MLORA_MAX_RANK) return fail(MLORA_ERANGE, "rank must be in 1..%d (got %d)", MLORA_MAX_RANK, r);
    int rc = check_dims(hin, hout);
    if (rc) return rc;
    if (!aligned16(y) || !aligned16(x) || !aligned16(wa_T_all) || !aligned16(wb_T_all))
        return fail(MLORA_EALIGN, "device pointers must be 16-byte aligned");
    if ((int64_t)N * L * r > 0x7fffffffLL) return fail(MLORA_ERANGE, "pool has more than 2^31-1 rank rows");
    mlora::BgmvArgs a;
    memset(&a, 0, sizeof(a));
    mlora::PoolView &pv = a.pool;
    pv.a_tbl = nullptr; pv.b_tbl = nullptr; pv.rank = nullptr; pv.scaling = nullptr;
    pv.n_adapters = N; pv.max_pages = 1; pv.page_shift = 0;
    pv.uniform_rank = r; pv.uniform_scale = scale;
    // A: rank rows of adapter i, layer l start at row (i*L + l)*r; the layer offset goes into the base pointer.
    pv.a_dense_stride = (long long)L * r;
    pv.n_rows_a = (long long)(N - 1) * L * r + r;
    // B^T: [hout, r] block of adapter i, layer l starts at element (i*L + l)*hout*r.
    pv.b_dense_stride = (long long)L * hout * r;
    pv.n_rows_b = 0;
    a.y[0] = y; a.x[0] = x;
    a.a_rows[0] = static_cast<const uint16_t *>(wa_T_all) + (size_t)layer_idx * r * hin;
    a.b_rows[0] = static_cast<const uint16_t *>(wb_T_all) + (size_t)layer_idx * hout * r;
    if (!aligned16(a.a_rows[0]) || !aligned16(a.b_rows[0]))
        return fail(MLORA_EALIGN, "layer slab of the pool is not 16-byte aligned (r * hin and hout * r must be multiples of 8)");
    a.hin[0] = hin; a.hout[0] = hout;
    a.tok_adapter = nullptr; a.tok_adapter64 = indices;
    a.T = T; a.n_proj = 1; a.accumulate = 1;
    rc = mlora::launch_bgmv(a, dtype, 1, r, true, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "bgmv launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

// Plan buffer of the reference-layout decode call: perm, seg_start, seg_len, seg_adapter, chunk_start, chunk_len,
// chunk_adapter (T int32 each, padded to 16 bytes), counters, then the work records.
static int64_t ref_plan_words(int T) { return ((int64_t)T + 3) / 4 * 4; }

int64_t mlora_reflayout_plan_bytes(int T)
{
    if (T <= 0) return 0;
    return (7 * ref_plan_words(T) + MLORA_CNT_WORDS + (int64_t)MLORA_WORK_CAP(T) * MLORA_WORK_WORDS) * (int64_t)sizeof(int32_t);
}

static int32_t *ref_plan_work(void *plan, int T) { return static_cast<int32_t *>(plan) + 7 * ref_plan_words(T) + MLORA_CNT_WORDS; }

static int ref_rank_ok(int r) { return r == 8 || r == 16 || r == 32 || r == 64; }

int mlora_reflayout_plan(const int64_t *indices, int T, int N, int L, int r, int group, void *plan, int64_t plan_bytes,
                         void *stream)
{
    if (T < 0) return fail(MLORA_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_OK;
    if (!indices || !plan) return fail(MLORA_EINVAL, "NULL pointer");
    if (T > MLORA_GATHER_MAX_T) return fail(MLORA_ERANGE, "T = %d exceeds MLORA_GATHER_MAX_T = %d", T, MLORA_GATHER_MAX_T);
    if (N <= 0 || N > (1 << 18) || L <= 0) return fail(MLORA_ERANGE, "N must be in 1..262144 and L positive (got %d, %d)", N, L);
    if (!ref_rank_ok(r)) return fail(MLORA_ERANGE, "the grouped reference-layout call needs rank 8, 16, 32 or 64 (got %d); mlora_bgmv_reflayout takes any rank", r);
    if (group != 1 && group != 2 && group != 4) return fail(MLORA_EINVAL, "group must be 1, 2 or 4 (got %d)", group);
    if ((int64_t)N * L * r > 0x7fffffffLL) return fail(MLORA_ERANGE, "pool has more than 2^31-1 rank rows");
    if (!aligned16(plan)) return fail(MLORA_EALIGN, "plan buffer must be 16-byte aligned");
    if (plan_bytes < mlora_reflayout_plan_bytes(T))
        return fail(MLORA_ENOSPACE, "plan buffer holds %lld bytes, %lld needed", (long long)plan_bytes, (long long)mlora_reflayout_plan_bytes(T));
    mlora::GatherArgs a;
    memset(&a, 0, sizeof(a));
    int32_t *ip = static_cast<int32_t *>(plan);
    const int64_t w = ref_plan_words(T);
    a.tok_adapter64 = indices;
    a.T = T; a.n_adapters = N; a.max_pages = 1; a.page_rows = 1; a.group = group;
    // rank row j of adapter a, relative to a layer's first row: a * L * r + j (wa_T_all is [N, L, r, hin])
    a.dense_stride = (long long)L * r; a.n_rows_dense = (long long)(N - 1) * L * r + r;
    a.uniform_rank = r; a.uniform_scale = 1.0f;
    a.perm = ip; a.seg_start = ip + w; a.seg_len = ip + 2 * w; a.seg_adapter = ip + 3 * w;
    a.chunk_start = ip + 4 * w; a.chunk_len = ip + 5 * w; a.chunk_adapter = ip + 6 * w; a.counters = ip + 7 * w;
    a.n_pages = 1; a.work = ref_plan_work(plan, T); a.work_cap = MLORA_WORK_CAP(T);
    const int rc = mlora::launch_gather(a, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "gather launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_bgmv_reflayout_multi(int n_proj, void *const *y, const void *const *x, const void *const *wa_T_all,
                               const void *const *wb_T_all, const int32_t *hin, const int32_t *hout, const void *plan,
                               int T, int N, int L, int r, int layer_idx, float scale, int group, int dtype,
                               int accumulate, void *workspace, int64_t workspace_bytes, void *stream)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (n_proj < 1 || n_proj > MLORA_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", MLORA_MAX_PROJ, n_proj);
    if (T < 0) return fail(MLORA_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_OK;
    if (!y || !x || !wa_T_all || !wb_T_all || !hin || !hout || !plan) return fail(MLORA_EINVAL, "NULL pointer");
    if (N <= 0 || L <= 0) return fail(MLORA_EINVAL, "N and L must be positive (got %d, %d)", N, L);
    if (layer_idx < 0 || layer_idx >= L) return fail(MLORA_ERANGE, "layer_idx %d outside [0, %d)", layer_idx, L);
    if (!ref_rank_ok(r)) return fail(MLORA_ERANGE, "the grouped reference-layout call needs rank 8, 16, 32 or 64 (got %d); mlora_bgmv_reflayout takes any rank", r);
    if (group != 1 && group != 2 && group != 4) return fail(MLORA_EINVAL, "group must be 1, 2 or 4 (got %d)", group);
    if ((int64_t)N * L * r > 0x7fffffffLL) return fail(MLORA_ERANGE, "pool has more than 2^31-1 rank rows");
    if (!aligned16(plan)) return fail(MLORA_EALIGN, "plan buffer must be 16-byte aligned");
    mlora::BgmvArgs a;
    memset(&a, 0, sizeof(a));
    mlora::PoolView &pv = a.pool;
    pv.n_adapters = N; pv.max_pages = 1; pv.page_shift = 0;
    pv.uniform_rank = r; pv.uniform_scale = scale;
    pv.a_dense_stride = (long long)L * r;
    pv.n_rows_a = (long long)(N - 1) * L * r + r;
    int max_hin = 0, max_hout = 0;
    for (int p = 0; p < n_proj; p++) {
        if (!y[p] || !x[p] || !wa_T_all[p] || !wb_T_all[p]) return fail(MLORA_EINVAL, "projection %d: NULL device pointer", p);
        int rc = check_dims(hin[p], hout[p]);
        if (rc) return rc;
        a.y[p] = y[p]; a.x[p] = x[p];
        a.a_rows[p] = static_cast<const uint16_t *>(wa_T_all[p]) + (size_t)layer_idx * r * hin[p];
        a.b_rows[p] = static_cast<const uint16_t *>(wb_T_all[p]) + (size_t)layer_idx * hout[p] * r;
        if (!aligned16(a.y[p]) || !aligned16(a.x[p]) || !aligned16(a.a_rows[p]) || !aligned16(a.b_rows[p]))
            return fail(MLORA_EALIGN, "projection %d: device pointers must be 16-byte aligned", p);
        a.hin[p] = hin[p]; a.hout[p] = hout[p];
        max_hin = hin[p] > max_hin ? hin[p] : max_hin;
        max_hout = hout[p] > max_hout ? hout[p] : max_hout;
    }
    a.b_transposed = 1; a.ref_layers = L;
    a.tok_adapter = nullptr; a.tok_adapter64 = nullptr;
    a.work = ref_plan_work(const_cast<void *>(plan), T); a.work_cap = MLORA_WORK_CAP(T);
    {
        const int64_t segs = T < N ? T : N;
        const int64_t bound = ((int64_t)(T + group - 1) / group + segs + 1 + 7) / 8 * 8;
        a.items_cap = bound < a.work_cap ? (int)bound : a.work_cap;
    }
    a.T = T; a.n_proj = n_proj; a.accumulate = accumulate ? 1 : 0;
    const int64_t need = mlora_bgmv_workspace_bytes(n_proj, T, max_hin, r);
    if (!workspace || !aligned16(workspace)) return fail(MLORA_EALIGN, "workspace must be a 16-byte aligned device pointer");
    if (workspace_bytes < need) return fail(MLORA_ENOSPACE, "workspace holds %lld bytes, %lld needed", (long long)workspace_bytes, (long long)need);
    a.vws = static_cast<float *>(workspace);
    int ksc, nte;
    mlora::bgmv_split_slices(r, &ksc, &nte, true);
    a.ks_max = (max_hin + ksc * 8 - 1) / (ksc * 8);
    a.cs_max = (max_hout + nte * 8 - 1) / (nte * 8);
    int sh = 0, ex = 0;
    for (int p = 0; p < n_proj; p++) {
        sh += (hin[p] + ksc * 8 - 1) / (ksc * 8);
        ex += (hout[p] + nte * 8 - 1) / (nte * 8);
        a.sh_end[p] = sh; a.ex_end[p] = ex;
    }
    const int rc = mlora::launch_bgmv_split(a, dtype, group, r, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "bgmv launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

}  // extern "C"

namespace {

constexpr int SG_TM = 64;   // tokens per tile, as in sgmv_prefill.hip

struct SgmvWs { int max_tiles; int ksplit; int ks_cap; size_t off_cover, off_rec, off_proj, per_proj, off_hi, off_lo, total; };

// Workspace: the plan (tile list, tile records: depends on T and n_seg only), then per projection the
// K-split partial sums and the hi / lo halves of their sum.
SgmvWs sgmv_layout(int T, int n_seg, int n_proj)
{
    SgmvWs w;
    w.max_tiles = T / SG_TM + 2 * n_seg + 1;       // aligned cuts can add one partial tile at either end of a segment
    // shrink workgroups: about three per CU for a single projection; a call over several projections has about
    // that many with one or two splits already (one workgroup serves the projections that share x), and fewer
    // splits mean less partial-sum traffic (swept 512 .. 4096 on configs 4 and 5: 768 - 1024 is the flat optimum)
    const long long per_split = (long long)w.max_tiles * n_proj;
    const long long target = n_proj > 1 ? 1024 : 768;
    long long ks = (target + per_split - 1) / per_split;
    w.ksplit = ks < 1 ? 1 : (ks > 8 ? 8 : (int)ks);
    // a projection with a longer K than the others of its call gets proportionally more splits (up to three
    // times as many, at most 8), so that every shrink workgroup walks about the same number of columns
    w.ks_cap = n_proj > 1 ? (3 * w.ksplit < 8 ? 3 * w.ksplit : 8) : w.ksplit;
    size_t off = ((size_t)w.max_tiles * 3 + 4) * sizeof(int32_t);
    off = (off + 255) & ~(size_t)255;
    w.off_cover = off;                              // int32 [T]: 1 where a token belongs to some segment
    off += (size_t)T * sizeof(int32_t);
    off = (off + 255) & ~(size_t)255;
    w.off_rec = off;
    off += (size_t)w.max_tiles * 80 * sizeof(int32_t);
    off = (off + 255) & ~(size_t)255;
    w.off_proj = off;
    w.off_hi = (size_t)w.ks_cap * T * MLORA_MAX_RANK * sizeof(float);
    w.off_lo = w.off_hi + (size_t)T * MLORA_MAX_RANK * sizeof(uint16_t);
    w.per_proj = (w.off_lo + (size_t)T * MLORA_MAX_RANK * sizeof(uint16_t) + 255) & ~(size_t)255;
    w.total = off + w.per_proj * n_proj;
    return w;
}

// Columns of y one expand workgroup covers, and the column blocks per tile that follow from it.
// 512 columns amortise the V operand; fewer when that leaves the chip idle (single-projection calls), and a block
// count per tile that the tile-major order of the expand can use (a multiple of eight or just below one):
// otherwise the width that gives the nearest multiple of eight blocks, in whole cache lines.
int expand_block_cols(int n_proj, int max_tiles, int hout, int *ncb_out)
{
    int cols = 512;
    if (n_proj == 1)
        while (cols > 128 && (long long)max_tiles * ((hout + cols - 1) / cols) < 1024) cols >>= 1;
    int ncb = (hout + cols - 1) / cols;
    if (!mlora::tile_major(ncb) && ncb >= 6) {
        const int n8 = ((ncb + 3) / 8) * 8 > 0 ? ((ncb + 3) / 8) * 8 : 8;
        const int c8 = ((hout + n8 - 1) / n8 + 63) / 64 * 64;
        if (c8 >= 256 && c8 <= 1024 && mlora::tile_major((hout + c8 - 1) / c8)) { cols = c8; ncb = (hout + c8 - 1) / c8; }
    }
    if (ncb_out) *ncb_out = ncb;
    return cols;
}

void carve(mlora::SgmvArgs &a, void *workspace, const SgmvWs &w)
{
    char *base = static_cast<char *>(workspace);
    int32_t *ip = reinterpret_cast<int32_t *>(base);
    a.tile_seg = ip; a.tile_tok0 = ip + w.max_tiles; a.tile_ntok = ip + 2 * (size_t)w.max_tiles;
    a.n_tiles = ip + 3 * (size_t)w.max_tiles;
    a.tok_cover = reinterpret_cast<int32_t *>(base + w.off_cover);
    a.tile_rec = reinterpret_cast<int32_t *>(base + w.off_rec);
    a.max_tiles = w.max_tiles;
    int hin_min = a.pr[0].hin;
    for (int p = 1; p < a.n_proj; p++) hin_min = a.pr[p].hin < hin_min ? a.pr[p].hin : hin_min;
    for (int p = 0; p < a.n_proj; p++) {
        char *pb = base + w.off_proj + w.per_proj * p;
        a.pr[p].v = reinterpret_cast<float *>(pb);
        a.pr[p].vhi = reinterpret_cast<uint16_t *>(pb + w.off_hi);
        a.pr[p].vlo = reinterpret_cast<uint16_t *>(pb + w.off_lo);
        int ks = (int)(((long long)w.ksplit * a.pr[p].hin + hin_min / 2) / (hin_min > 0 ? hin_min : 1));
        a.pr[p].ksplit = ks < w.ksplit ? w.ksplit : (ks > w.ks_cap ? w.ks_cap : ks);
        int ncb = 0;
        const int cols = expand_block_cols(a.n_proj, w.max_tiles, a.pr[p].hout, &ncb);
        a.pr[p].cols = cols;
        a.pr[p].ncb = ncb;
    }
    // shrink groups: up to three consecutive projections that read the same activations (one workgroup serves a group)
    a.n_grp = 0;
    for (int p = 0; p < a.n_proj; p++) {
        if (p > 0 && a.pr[p].x == a.pr[p - 1].x && a.pr[p].hin == a.pr[p - 1].hin && a.grp_n[a.n_grp - 1] < 3) a.grp_n[a.n_grp - 1]++;
        else { a.grp_first[a.n_grp] = p; a.grp_n[a.n_grp] = 1; a.n_grp++; }
    }
}

}  // namespace

extern "C" {

int64_t mlora_sgmv_workspace_bytes(int T, int n_seg)
{
    if (T <= 0 || n_seg <= 0) return 256;
    return (int64_t)sgmv_layout(T, n_seg, 1).total;
}

int mlora_sgmv_expand_cols(int T, int n_seg, int n_proj, int hout)
{
    if (T <= 0 || n_seg <= 0 || n_proj < 1 || n_proj > MLORA_MAX_PROJ || hout <= 0) return 0;
    return expand_block_cols(n_proj, sgmv_layout(T, n_seg, n_proj).max_tiles, hout, nullptr);
}

int64_t mlora_sgmv_multi_workspace_bytes(int T, int n_seg, int n_proj)
{
    if (T <= 0 || n_seg <= 0 || n_proj < 1 || n_proj > MLORA_MAX_PROJ) return 256;
    return (int64_t)sgmv_layout(T, n_seg, n_proj).total;
}

static int sgmv_common(int n_proj, void *const *y, const void *const *x, const void *const *a_rows,
                       const void *const *b_rows, const int32_t *hin, const int32_t *hout, const int32_t *seg_start,
                       const int32_t *seg_len, const int32_t *seg_adapter, int n_seg, const int32_t *page_tbl,
                       const int32_t *rank, const float *scaling, int T, int n_adapters,
                       int max_pages, int page_rows, int64_t n_pages, int max_rank, int dtype, int accumulate,
                       void *workspace, int64_t workspace_bytes, int phases, void *stream, int tile_aligned = 0)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (T < 0 || n_seg < 0) return fail(MLORA_EINVAL, "T and n_seg must be >= 0 (got %d, %d)", T, n_seg);
    if (n_proj < 1 || n_proj > MLORA_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", MLORA_MAX_PROJ, n_proj);
    if (T == 0 || n_seg == 0) return MLORA_OK;
    if (!seg_start || !seg_len || !seg_adapter) return fail(MLORA_EINVAL, "NULL device pointer");
    mlora::SgmvArgs a;
    memset(&a, 0, sizeof(a));
    int rc = check_pool(a.pool, page_tbl, rank, scaling, n_adapters, max_pages, page_rows, n_pages, max_rank);
    if (rc) return rc;
    a.n_proj = n_proj;
    if (phases & mlora::SGMV_APPLY) {
        if (!y || !x || !a_rows || !b_rows || !hin || !hout) return fail(MLORA_EINVAL, "per-projection arrays must not be NULL");
        for (int p = 0; p < n_proj; p++) {
            if (!y[p] || !x[p] || !a_rows[p] || !b_rows[p]) return fail(MLORA_EINVAL, "projection %d: NULL device pointer", p);
            rc = check_dims(hin[p], hout[p]);
            if (rc) return rc;
            if (!aligned16(y[p]) || !aligned16(x[p]) || !aligned16(a_rows[p]) || !aligned16(b_rows[p]))
                return fail(MLORA_EALIGN, "projection %d: device pointers must be 16-byte aligned", p);
            a.pr[p].y = y[p]; a.pr[p].x = x[p]; a.pr[p].a_rows = a_rows[p]; a.pr[p].b_rows = b_rows[p];
            a.pr[p].hin = hin[p]; a.pr[p].hout = hout[p];
        }
    } else {
        a.pr[0].hin = 8; a.pr[0].hout = 8;
    }
    const SgmvWs w = sgmv_layout(T, n_seg, n_proj);
    if (!workspace || !aligned16(workspace)) return fail(MLORA_EALIGN, "workspace must be a 16-byte aligned device pointer");
    if (workspace_bytes < (int64_t)w.total)
        return fail(MLORA_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)w.total);
    a.seg_start = seg_start; a.seg_len = seg_len; a.seg_adapter = seg_adapter; a.n_seg = n_seg;
    a.T = T; a.accumulate = accumulate ? 1 : 0; a.b_transposed = 0; a.seg_uniform_len = 0; a.tile_aligned = tile_aligned;
    carve(a, workspace, w);
    rc = mlora::launch_sgmv(a, dtype, max_rank, phases, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "sgmv launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_sgmv(void *y, const void *x, const void *a_rows, const void *b_rows, const int32_t *seg_start,
               const int32_t *seg_len, const int32_t *seg_adapter, int n_seg, const int32_t *page_tbl,
               const int32_t *rank, const float *scaling, int T, int hin, int hout,
               int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
               int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream)
{
    void *ys[1] = {y};
    const void *xs[1] = {x}, *as[1] = {a_rows}, *bs[1] = {b_rows};
    const int32_t hi[1] = {hin}, ho[1] = {hout};
    return sgmv_common(1, ys, xs, as, bs, hi, ho, seg_start, seg_len, seg_adapter, n_seg, page_tbl, rank, scaling, T,
                       n_adapters, max_pages, page_rows, n_pages, max_rank, dtype, accumulate, workspace,
                       workspace_bytes, mlora::SGMV_PLAN | mlora::SGMV_APPLY, stream);
}

int mlora_sgmv_plan(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                    const int32_t *page_tbl, const int32_t *rank, const float *scaling, int T, int n_adapters,
                    int max_pages, int page_rows, int64_t n_pages, int max_rank, void *workspace,
                    int64_t workspace_bytes, void *stream)
{
    return sgmv_common(1, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, seg_start, seg_len, seg_adapter, n_seg,
                       page_tbl, rank, scaling, T, n_adapters, max_pages, page_rows, n_pages, max_rank, MLORA_F16, 0,
                       workspace, workspace_bytes, mlora::SGMV_PLAN, stream);
}

int mlora_sgmv_plan_aligned(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                            const int32_t *page_tbl, const int32_t *rank, const float *scaling, int T, int n_adapters,
                            int max_pages, int page_rows, int64_t n_pages, int max_rank, void *workspace,
                            int64_t workspace_bytes, void *stream)
{
    return sgmv_common(1, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, seg_start, seg_len, seg_adapter, n_seg,
                       page_tbl, rank, scaling, T, n_adapters, max_pages, page_rows, n_pages, max_rank, MLORA_F16, 0,
                       workspace, workspace_bytes, mlora::SGMV_PLAN, stream, 1);
}

int mlora_sgmv_planned(void *y, const void *x, const void *a_rows, const void *b_rows, const int32_t *seg_start,
                       const int32_t *seg_len, const int32_t *seg_adapter, int n_seg, const int32_t *page_tbl,
                       const int32_t *rank, const float *scaling, int T, int hin, int hout,
                       int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                       int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream)
{
    void *ys[1] = {y};
    const void *xs[1] = {x}, *as[1] = {a_rows}, *bs[1] = {b_rows};
    const int32_t hi[1] = {hin}, ho[1] = {hout};
    return sgmv_common(1, ys, xs, as, bs, hi, ho, seg_start, seg_len, seg_adapter, n_seg, page_tbl, rank, scaling, T,
                       n_adapters, max_pages, page_rows, n_pages, max_rank, dtype, accumulate, workspace,
                       workspace_bytes, mlora::SGMV_APPLY, stream);
}

int mlora_sgmv_multi_planned(int n_proj, void *const *y, const void *const *x, const void *const *a_rows,
                             const void *const *b_rows, const int32_t *hin, const int32_t *hout,
                             const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter, int n_seg,
                             const int32_t *page_tbl, const int32_t *rank, const float *scaling, int T,
                             int n_adapters, int max_pages, int page_rows, int64_t n_pages, int max_rank,
                             int dtype, int accumulate, void *workspace, int64_t workspace_bytes, void *stream)
{
    return sgmv_common(n_proj, y, x, a_rows, b_rows, hin, hout, seg_start, seg_len, seg_adapter, n_seg, page_tbl, rank,
                       scaling, T, n_adapters, max_pages, page_rows, n_pages, max_rank, dtype, accumulate, workspace,
                       workspace_bytes, mlora::SGMV_APPLY, stream);
}

int mlora_gemm_lora_planned(int n_proj, void *const *y, const void *const *x, const void *const *w,
                            const void *const *a_rows, const void *const *b_rows, const int32_t *hin,
                            const int32_t *hout, const int32_t *seg_start, const int32_t *seg_len,
                            const int32_t *seg_adapter, int n_seg, const int32_t *page_tbl, const int32_t *rank,
                            const float *scaling, int T, int n_adapters, int max_pages, int page_rows,
                            int64_t n_pages, int max_rank, int dtype, void *workspace, int64_t workspace_bytes,
                            void *stream)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (T < 0 || n_seg < 0) return fail(MLORA_EINVAL, "T and n_seg must be >= 0 (got %d, %d)", T, n_seg);
    if (n_proj < 1 || n_proj > MLORA_MAX_PROJ) return fail(MLORA_ERANGE, "n_proj must be in 1..%d (got %d)", MLORA_MAX_PROJ, n_proj);
    if (T == 0) return MLORA_OK;
    if (!y || !x || !w || !hin || !hout) return fail(MLORA_EINVAL, "per-projection arrays must not be NULL");
    const bool lora = n_seg > 0;
    if (lora && (!a_rows || !b_rows || !seg_start || !seg_len || !seg_adapter)) return fail(MLORA_EINVAL, "NULL pointer for a call with segments");
    mlora::SgmvArgs a;
    memset(&a, 0, sizeof(a));
    mlora::GemmLoraArgs g;
    memset(&g, 0, sizeof(g));
    int rc;
    if (lora) {
        rc = check_pool(a.pool, page_tbl, rank, scaling, n_adapters, max_pages, page_rows, n_pages, max_rank);
        if (rc) return rc;
    }
    a.n_proj = n_proj;
    for (int p = 0; p < n_proj; p++) {
        if (!y[p] || !x[p] || !w[p] || (lora && (!a_rows[p] || !b_rows[p]))) return fail(MLORA_EINVAL, "projection %d: NULL device pointer", p);
        rc = check_dims(hin[p], hout[p]);
        if (rc) return rc;
        if (!aligned16(y[p]) || !aligned16(x[p]) || !aligned16(w[p]) || (lora && (!aligned16(a_rows[p]) || !aligned16(b_rows[p]))))
            return fail(MLORA_EALIGN, "projection %d: device pointers must be 16-byte aligned", p);
        // the kernel addresses a weight through one buffer descriptor with 32-bit offsets
        if ((int64_t)hin[p] * hout[p] * 2 >= (1LL << 32)) return fail(MLORA_ERANGE, "projection %d: base weight of 4 GiB or more", p);
        if ((int64_t)256 * hin[p] * 2 >= (1LL << 32)) return fail(MLORA_ERANGE, "projection %d: hin too large", p);
        a.pr[p].y = y[p]; a.pr[p].x = x[p]; a.pr[p].hin = hin[p]; a.pr[p].hout = hout[p];
        g.pr[p].y = y[p]; g.pr[p].x = x[p]; g.pr[p].w = w[p]; g.pr[p].hin = hin[p]; g.pr[p].hout = hout[p];
        if (lora) {
            a.pr[p].a_rows = a_rows[p]; a.pr[p].b_rows = b_rows[p]; g.pr[p].b_rows = b_rows[p];
            // the B rows slab is addressed through one descriptor as well
            if ((int64_t)a.pool.n_rows_b * hout[p] * 2 >= 0xfff00000LL) return fail(MLORA_ERANGE, "projection %d: B rows slab of 4 GiB or more", p);
        }
    }
    g.n_proj = n_proj; g.T = T; g.lora = lora ? 1 : 0;
    if (lora) {
        const SgmvWs ws = sgmv_layout(T, n_seg, n_proj);
        if (!workspace || !aligned16(workspace)) return fail(MLORA_EALIGN, "workspace must be a 16-byte aligned device pointer");
        if (workspace_bytes < (int64_t)ws.total)
            return fail(MLORA_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)ws.total);
        a.seg_start = seg_start; a.seg_len = seg_len; a.seg_adapter = seg_adapter; a.n_seg = n_seg;
        a.T = T; a.accumulate = 0; a.b_transposed = 0; a.seg_uniform_len = 0;
        carve(a, workspace, ws);
        rc = mlora::launch_sgmv(a, dtype, max_rank, mlora::SGMV_SHRINK, static_cast<hipStream_t>(stream));
        if (rc) return fail(MLORA_ELAUNCH, "shrink launch failed: %s", hipGetErrorString((hipError_t)rc));
        for (int p = 0; p < n_proj; p++) {
            g.pr[p].v = a.pr[p].v; g.pr[p].vhi = a.pr[p].vhi; g.pr[p].vlo = a.pr[p].vlo; g.pr[p].ksplit = a.pr[p].ksplit;
        }
        g.tile_rec = a.tile_rec; g.n_tiles = a.n_tiles; g.max_tiles = a.max_tiles; g.n_rows_b = a.pool.n_rows_b;
    }
    rc = mlora::launch_gemm_lora(g, dtype, lora ? max_rank : 16, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "gemm launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

int mlora_prefill_reflayout(void *y, const void *x, const void *A_T, const void *B_T, int B, int Lpad, int L,
                            int r, int hin, int hout, int layer_idx, int dtype, void *workspace,
                            int64_t workspace_bytes, void *stream)
{
    if (dtype != MLORA_F16 && dtype != MLORA_BF16) return fail(MLORA_EDTYPE, "dtype must be MLORA_F16 or MLORA_BF16 (got %d)", dtype);
    if (B < 0 || Lpad < 0) return fail(MLORA_EINVAL, "B and Lpad must be >= 0 (got %d, %d)", B, Lpad);
    if (B == 0 || Lpad == 0) return MLORA_OK;
    if ((int64_t)B * Lpad > 0x7fffffffLL) return fail(MLORA_ERANGE, "B * Lpad exceeds 2^31-1 tokens");
    if (!y || !x || !A_T || !B_T) return fail(MLORA_EINVAL, "NULL device pointer");
    if (L <= 0 || layer_idx < 0 || layer_idx >= L) return fail(MLORA_ERANGE, "layer_idx %d outside [0, %d)", layer_idx, L);
    if (r < 8 || r > MLORA_MAX_RANK || (r & 7)) return fail(MLORA_ERANGE, "prefill on the reference layout needs a rank that is a multiple of 8 in 8..%d (got %d)", MLORA_MAX_RANK, r);
    int rc = check_dims(hin, hout);
    if (rc) return rc;
    if (!aligned16(y) || !aligned16(x) || !aligned16(A_T) || !aligned16(B_T))
        return fail(MLORA_EALIGN, "device pointers must be 16-byte aligned");
    if ((int64_t)B * L * r > 0x7fffffffLL) return fail(MLORA_ERANGE, "pool has more than 2^31-1 rank rows");
    const int T = B * Lpad;
    const SgmvWs w = sgmv_layout(T, B, 1);
    if (!workspace || !aligned16(workspace)) return fail(MLORA_EALIGN, "workspace must be a 16-byte aligned device pointer");
    if (workspace_bytes < (int64_t)w.total)
        return fail(MLORA_ENOSPACE, "workspace has %lld bytes, %lld needed", (long long)workspace_bytes, (long long)w.total);
    mlora::SgmvArgs a;
    memset(&a, 0, sizeof(a));
    mlora::PoolView &pv = a.pool;
    pv.n_adapters = B; pv.max_pages = 1; pv.page_shift = 0;
    pv.uniform_rank = r; pv.uniform_scale = 1.0f;
    pv.a_dense_stride = (long long)L * r;
    pv.n_rows_a = (long long)(B - 1) * L * r + r;
    pv.b_dense_stride = (long long)L * hout * r;
    pv.n_rows_b = 0;
    a.n_proj = 1;
    a.pr[0].y = y; a.pr[0].x = x;
    a.pr[0].a_rows = static_cast<const uint16_t *>(A_T) + (size_t)layer_idx * r * hin;
    a.pr[0].b_rows = static_cast<const uint16_t *>(B_T) + (size_t)layer_idx * hout * r;
    a.pr[0].hin = hin; a.pr[0].hout = hout;
    a.n_seg = B; a.T = T; a.accumulate = 0; a.b_transposed = 1; a.seg_uniform_len = Lpad;
    carve(a, workspace, w);
    rc = mlora::launch_sgmv(a, dtype, r, mlora::SGMV_PLAN | mlora::SGMV_APPLY, static_cast<hipStream_t>(stream));
    if (rc) return fail(MLORA_ELAUNCH, "prefill launch failed: %s", hipGetErrorString((hipError_t)rc));
    return MLORA_OK;
}

}  // extern "C"
