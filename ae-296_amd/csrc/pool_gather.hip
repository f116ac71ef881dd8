// Adapter-pool index/offset gather for gfx950.
//
// Block 0 groups the tokens of a batch by adapter (stable: ordered by adapter id, then by
// token id) with a bitonic sort of 32-bit keys in LDS, and derives segments and the decode
// work list (chunks of at most `group` tokens of one adapter) with block-wide scans.
// Blocks 1.. write the per-token view: page base rows, rank and scaling of each token's
// adapter.  All outputs are integers or copied floats, so they are bit-exact by construction.
//
// Stands where the reference draws / selects its per-token index vector
// (lightllm/models/lora_gpu.py:120,124,143,155) and drops the real per-request ids
// (lightllm/server/router/model_infer/pre_process.py:50,100).
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

constexpr int GATHER_NT_MAX = 1024;
constexpr int GATHER_MAX_T = 8192;
constexpr int TOK_BITS = 13;                 // token id field of the sort key

// Adapter id of token i as the kernels see it: negative = none, >= n_adapters = out of range (counted, then none).
// An int64 id (the reference's index vector) outside [0, n_adapters) is "none" on either side.
__device__ __forceinline__ int gather_adapter(const GatherArgs &g, int i)
{
    if (g.tok_adapter) return g.tok_adapter[i];
    const long long a = g.tok_adapter64[i];
    return a < 0 ? -1 : (a >= g.n_adapters ? g.n_adapters : (int)a);
}
__device__ __forceinline__ int gather_rank(const GatherArgs &g, int a) { return g.rank ? g.rank[a] : g.uniform_rank; }
__device__ __forceinline__ float gather_scale(const GatherArgs &g, int a) { return g.scaling ? g.scaling[a] : g.uniform_scale; }
// Row (in a rows slab) of rank row j of adapter a, -1 if it does not exist.
__device__ __forceinline__ int gather_row(const GatherArgs &g, int a, int j)
{
    if (!g.page_tbl) {
        const long long row = (long long)a * g.dense_stride + j;
        return row < g.n_rows_dense ? (int)row : -1;
    }
    if (j / g.page_rows >= g.max_pages) return -1;
    const int pg = g.page_tbl[(long long)a * g.max_pages + j / g.page_rows];
    return (pg >= 0 && pg < g.n_pages) ? pg * g.page_rows + j % g.page_rows : -1;
}

// Inclusive scan over the block's per-thread values; op = 0 sum, 1 max, 2 min.
template <int OP>
__device__ __forceinline__ int scan_op(int a, int b)
{
    if constexpr (OP == 0) return a + b;
    else if constexpr (OP == 1) return a > b ? a : b;
    else return a < b ? a : b;
}

template <int OP>
__device__ int block_scan_inclusive(int v, int identity, int *s_wave /* [16] */)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(v, d);
        if (lane >= d) v = scan_op<OP>(v, o);
    }
    __syncthreads();                 // s_wave may still be read by a previous scan
    if (lane == 63) s_wave[wave] = v;
    __syncthreads();
    int base = identity;
    for (int w = 0; w < wave; w++) base = scan_op<OP>(base, s_wave[w]);
    return scan_op<OP>(base, v);
}

// One workgroup of GATHER_NT threads groups up to MAXT tokens (EPT sorted positions per thread in the
// scans).  The MAXT = 2048 instance also keeps the chunk headers in LDS, which makes writing the work
// records cheap; decode batches are normally that small.
template <int GATHER_NT, int MAXT>
__global__ __launch_bounds__(GATHER_NT) void gather_kernel(const GatherArgs g)
{
    constexpr int EPT = MAXT / GATHER_NT;
    const int tid = threadIdx.x;
    if (blockIdx.x > 0) {
        // ---- per-token view
        const long long idx = (long long)(blockIdx.x - 1) * GATHER_NT + tid;
        const long long total = (long long)g.T * g.max_pages;
        if (idx >= total) return;
        const int t = (int)(idx / g.max_pages), pg = (int)(idx - (long long)t * g.max_pages);
        int a = gather_adapter(g, t);
        if (a >= g.n_adapters) a = -1;
        int r = 0;
        float s = 0.f;
        int off = -1;
        if (a >= 0) {
            r = g.rank[a];
            s = g.scaling[a];
            const int np = (r + g.page_rows - 1) / g.page_rows;
            if (pg < np) off = g.page_tbl[(long long)a * g.max_pages + pg] * g.page_rows;
        }
        if (g.out_row_off) g.out_row_off[idx] = off;
        if (pg == 0) {
            if (g.out_rank) g.out_rank[t] = r;
            if (g.out_scale) g.out_scale[t] = s;
        }
        return;
    }
    if (!g.perm) return;

    // ---- grouped view (one workgroup)
    constexpr bool LDS_HDR = MAXT <= 2048;                 // chunk headers fit in LDS next to the keys
    __shared__ uint32_t s_key[MAXT];
    __shared__ int s_chdr[LDS_HDR ? MAXT : 1];             // start | len << 13 | rank << 17 per chunk
    __shared__ float s_cscale[LDS_HDR ? MAXT : 1];
    __shared__ int s_wave[16];
    __shared__ int s_cnt[2];
    const int T = g.T;
    int n2 = 2;
    while (n2 < T) n2 <<= 1;
    if (tid < 2) s_cnt[tid] = 0;
    __syncthreads();
    const uint32_t sentinel = (uint32_t)g.n_adapters;   // "no adapter" sorts after every real adapter
    for (int i = tid; i < n2; i += GATHER_NT) {
        uint32_t key = 0xffffffffu;
        bool valid = false, bad = false;
        if (i < T) {
            const int a = gather_adapter(g, i);
            bad = a >= g.n_adapters;
            valid = a >= 0 && !bad;
            key = ((valid ? (uint32_t)a : sentinel) << TOK_BITS) | (uint32_t)i;
        }
        s_key[i] = key;
        const unsigned long long mv = __ballot(valid), mb = __ballot(bad);
        if ((tid & 63) == 0) {
            if (mv) atomicAdd(&s_cnt[0], __popcll(mv));
            if (mb) atomicAdd(&s_cnt[1], __popcll(mb));
        }
    }
    __syncthreads();
    for (int k = 2; k <= n2; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < (n2 >> 1); i += GATHER_NT) {
                const int lo = 2 * i - (i & (j - 1));
                const int hi = lo + j;
                const uint32_t a = s_key[lo], b = s_key[hi];
                const bool up = (lo & k) == 0;
                if ((a > b) == up) { s_key[lo] = b; s_key[hi] = a; }
            }
            __syncthreads();
        }
    }
    const int n_valid = s_cnt[0];
    const int gmask = g.group - 1;

    // Each thread owns EPT consecutive sorted positions.
    int ad[EPT], head[EPT];
    const int base = tid * EPT;
#pragma unroll
    for (int e = 0; e < EPT; e++) {
        const int i = base + e;
        ad[e] = -1; head[e] = 0;
        if (i < T) {
            const uint32_t key = s_key[i];
            ad[e] = (int)(key >> TOK_BITS);
            g.perm[i] = (int)(key & ((1u << TOK_BITS) - 1u));
            head[e] = (i == 0) || ((int)(s_key[i - 1] >> TOK_BITS) != ad[e]);
        }
    }
    // segment start of every position: running max of head positions
    int run = 0, segstart[EPT];
#pragma unroll
    for (int e = 0; e < EPT; e++) { if (head[e]) run = base + e; segstart[e] = run; }
    {
        const int incl = block_scan_inclusive<1>(run, 0, s_wave);
        const int prev = __shfl_up(incl, 1);          // exclusive value for this thread
        __syncthreads();
        if ((tid & 63) == 63) s_wave[tid >> 6] = incl;
        __syncthreads();
        int excl = (tid & 63) ? prev : ((tid >> 6) ? s_wave[(tid >> 6) - 1] : 0);
        bool seen = false;
#pragma unroll
        for (int e = 0; e < EPT; e++) { seen = seen || head[e]; if (!seen) segstart[e] = excl; }
    }
    // segment end of every position: next head position after it (T if none): reverse running min
    int segend[EPT];
    {
        int nxt = T;
        int own_first = T;                       // first head position inside this thread's range
#pragma unroll
        for (int e = EPT - 1; e >= 0; e--) { segend[e] = nxt; if (head[e]) nxt = base + e; }
        own_first = nxt;
        // suffix min over threads = prefix min over reversed thread order
        const int rt = GATHER_NT - 1 - tid;
        __syncthreads();
        __shared__ int s_first[GATHER_NT];
        s_first[rt] = own_first;
        __syncthreads();
        const int mine = s_first[tid];            // value of thread (NT-1-tid)
        const int incl = block_scan_inclusive<2>(mine, T, s_wave);
        __syncthreads();
        s_first[tid] = incl;                      // min over reversed index <= tid
        __syncthreads();
        const int after = rt > 0 ? s_first[rt - 1] : T;   // min over threads with larger tid
#pragma unroll
        for (int e = 0; e < EPT; e++) if (segend[e] == T) segend[e] = after < T ? after : T;
    }
    // running counts of real segment heads and of chunk heads
    int nseg_local = 0, nch_local = 0, chead[EPT];
#pragma unroll
    for (int e = 0; e < EPT; e++) {
        const int i = base + e;
        chead[e] = (i < T) && (((i - segstart[e]) & gmask) == 0);
        nseg_local += (head[e] && ad[e] < g.n_adapters) ? 1 : 0;
        nch_local += chead[e];
    }
    const int seg_incl = block_scan_inclusive<0>(nseg_local, 0, s_wave);
    const int ch_incl = block_scan_inclusive<0>(nch_local, 0, s_wave);
    int seg_idx = seg_incl - nseg_local, ch_idx = ch_incl - nch_local;
#pragma unroll
    for (int e = 0; e < EPT; e++) {
        const int i = base + e;
        const bool real = ad[e] >= 0 && ad[e] < g.n_adapters;
        if (head[e] && real) {
            g.seg_start[seg_idx] = i;
            g.seg_len[seg_idx] = segend[e] - i;
            g.seg_adapter[seg_idx] = ad[e];
            seg_idx++;
        }
        if (chead[e]) {
            const int left = segend[e] - i;
            const int len = left < g.group ? left : g.group;
            g.chunk_start[ch_idx] = i;
            g.chunk_len[ch_idx] = len;
            g.chunk_adapter[ch_idx] = real ? ad[e] : -1;
            if constexpr (LDS_HDR) {
                if (g.work) {
                    int rk = 0;
                    float sc = 0.f;
                    if (real) { rk = gather_rank(g, ad[e]); rk = rk < 0 ? 0 : (rk > MAX_RANK ? MAX_RANK : rk); sc = gather_scale(g, ad[e]); }
                    s_chdr[ch_idx] = i | (len << TOK_BITS) | (rk << (TOK_BITS + 4));
                    s_cscale[ch_idx] = sc;
                }
            }
            ch_idx++;
        }
    }
    // ---- decode work records, in launch order: the records in use first; records b, b + 8, ... hold consecutive
    // chunks (the one-launch decode form, whose workgroup b of a projection reads record b, runs them on one XCD:
    // workgroups are dealt to the 8 XCDs round-robin; the two-launch form takes the records in order).  Batches
    // beyond 2048 tokens (chunk headers not in LDS) keep plain chunk order inside each range.
    if (g.work) {
        __shared__ int s_nchunks;
        if (tid == GATHER_NT - 1) s_nchunks = ch_incl;
        __syncthreads();                         // chunk_* arrays written above are visible to the whole block
        const int n_chunks = s_nchunks;
        const int per_xcd = (n_chunks + 7) >> 3;
        if constexpr (LDS_HDR) {
            // Within each of the eight ranges of chunks the records are written in order of falling rank
            // (ties keep chunk order, so the chunks of one adapter stay next to each other): the workgroups of
            // the wide items are then dispatched first and the narrow ones fill in behind them.  A counting sort:
            // chunks per (XCD, rank), then one thread per (XCD, rank) places its chunks.
            __shared__ int s_ord[MAXT];
            __shared__ int s_cntx[8][MAX_RANK + 1];
            int differs = 0;                     // a pool of one rank keeps chunk order and skips the sort
            for (int c = tid; c < n_chunks; c += GATHER_NT) differs |= (s_chdr[c] >> (TOK_BITS + 4)) != (s_chdr[0] >> (TOK_BITS + 4));
            for (int i = tid; i < 8 * (MAX_RANK + 1); i += GATHER_NT) (&s_cntx[0][0])[i] = 0;
            const bool mixed = __syncthreads_or(differs) != 0;
            if (mixed)
                for (int c = tid; c < n_chunks; c += GATHER_NT) atomicAdd(&s_cntx[c / per_xcd][s_chdr[c] >> (TOK_BITS + 4)], 1);
            __syncthreads();
            if (mixed && tid < 8 * (MAX_RANK + 1)) {
                const int xcd = tid / (MAX_RANK + 1), rk = tid - xcd * (MAX_RANK + 1);
                if (s_cntx[xcd][rk] > 0) {
                    int at = xcd * per_xcd;
                    for (int r2 = rk + 1; r2 <= MAX_RANK; r2++) at += s_cntx[xcd][r2];
                    const int lo = xcd * per_xcd, hi = lo + per_xcd < n_chunks ? lo + per_xcd : n_chunks;
                    for (int c = lo; c < hi; c++)
                        if ((s_chdr[c] >> (TOK_BITS + 4)) == rk) s_ord[at++] = c;
                }
            }
            __syncthreads();
            // 16 bytes per step: header quad, two token quads, a zero quad, then 16 quads of row indices.
            constexpr int QPR = WORK_WORDS / 4;
            int4 *out = reinterpret_cast<int4 *>(g.work);
            const int quads = g.work_cap * QPR;
            const uint32_t tmask = (1u << TOK_BITS) - 1u;
#pragma unroll 4
            for (int q = tid; q < quads; q += GATHER_NT) {
                const int b = q / QPR, w4 = q - b * QPR;
                const int pos = (b & 7) * per_xcd + (b >> 3);
                int4 v = make_int4(0, w4 == 0 ? -1 : 0, 0, 0);
                if ((b >> 3) < per_xcd && pos < n_chunks) {
                    const int c = mixed ? s_ord[pos] : pos;
                    const int hdr = s_chdr[c];
                    const int start = hdr & (int)tmask, len = (hdr >> TOK_BITS) & 15, rk = hdr >> (TOK_BITS + 4);
                    int a = (int)(s_key[start] >> TOK_BITS);
                    a = a < g.n_adapters ? a : -1;
                    if (w4 == 0) v = make_int4(len, a, rk, __builtin_bit_cast(int, s_cscale[c]));
                    else if (w4 <= 2) {
                        const int k0 = (w4 - 1) * 4;
                        v.x = k0 + 0 < len ? (int)(s_key[start + k0 + 0] & tmask) : -1;
                        v.y = k0 + 1 < len ? (int)(s_key[start + k0 + 1] & tmask) : -1;
                        v.z = k0 + 2 < len ? (int)(s_key[start + k0 + 2] & tmask) : -1;
                        v.w = k0 + 3 < len ? (int)(s_key[start + k0 + 3] & tmask) : -1;
                    } else if (w4 >= WORK_ROWS_AT / 4) {
                        const int j0 = (w4 - WORK_ROWS_AT / 4) * 4;
                        int rr[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int j = j0 + e;
                            rr[e] = (a >= 0 && j < rk) ? gather_row(g, a, j) : -1;
                        }
                        v = make_int4(rr[0], rr[1], rr[2], rr[3]);
                    }
                }
                out[q] = v;
            }
        } else {
        const long long words = (long long)g.work_cap * WORK_WORDS;
        for (long long idx = tid; idx < words; idx += GATHER_NT) {
            const int b = (int)(idx / WORK_WORDS), w = (int)(idx - (long long)b * WORK_WORDS);
            const int c = (b & 7) * per_xcd + (b >> 3);
            int val = w == 1 ? -1 : 0;
            if ((b >> 3) < per_xcd && c < n_chunks) {
                const int start = g.chunk_start[c], len = g.chunk_len[c], a = g.chunk_adapter[c];
                int rk = 0;
                if (a >= 0) { rk = gather_rank(g, a); rk = rk < 0 ? 0 : (rk > MAX_RANK ? MAX_RANK : rk); }
                if (w == 0) val = len;
                else if (w == 1) val = a;
                else if (w == 2) val = rk;
                else if (w == 3) val = a >= 0 ? __builtin_bit_cast(int, gather_scale(g, a)) : 0;
                else if (w < 12) val = (w - 4) < len ? (int)(s_key[start + (w - 4)] & ((1u << TOK_BITS) - 1u)) : -1;
                else if (w < WORK_ROWS_AT) val = 0;
                else {
                    const int j = w - WORK_ROWS_AT;
                    val = (a >= 0 && j < rk) ? gather_row(g, a, j) : -1;
                }
            }
            g.work[idx] = val;
        }
        }
    }
    if (tid == GATHER_NT - 1) {
        g.counters[0] = seg_incl;
        g.counters[1] = n_valid;
        g.counters[2] = ch_incl;
        g.counters[3] = s_cnt[1];
        g.counters[4] = 0; g.counters[5] = 0; g.counters[6] = 0; g.counters[7] = 0;
    }
}

int launch_gather(const GatherArgs &a, hipStream_t s)
{
    const long long per_tok = (a.out_row_off || a.out_rank || a.out_scale) ? (long long)a.T * a.max_pages : 0;
    const unsigned grid = 1u + (unsigned)((per_tok + GATHER_NT_MAX - 1) / GATHER_NT_MAX);
    if (a.T <= 2048) hipLaunchKernelGGL((gather_kernel<GATHER_NT_MAX, 2048>), dim3(grid), dim3(GATHER_NT_MAX), 0, s, a);
    else hipLaunchKernelGGL((gather_kernel<GATHER_NT_MAX, GATHER_MAX_T>), dim3(grid), dim3(GATHER_NT_MAX), 0, s, a);
    return (int)hipGetLastError();
}

}  // namespace mlora
