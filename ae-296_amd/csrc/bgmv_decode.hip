// BGMV decode kernel for gfx950: y[t] (+)= s_a * (x[t] . A_a) . B_a, shrink and expand
// fused in one launch.  One workgroup owns one work item = up to G tokens that use the
// same adapter (G = 1: one token per workgroup), so an adapter's rows are fetched once
// per item and the rank-r intermediate never leaves the CU (fp32 in LDS).
//
// Work items come in two forms:
//   - work records written by the gather kernel (WORK = true): one 320-byte record per
//     workgroup holding the tokens, the adapter's rank, scaling and the row index of every
//     rank row, already placed in launch order -- one dependent load before the streaming
//     starts, no table walk, no barrier;
//   - the plain form (WORK = false): workgroup t serves token t and walks the page table
//     (or the dense reference layout) itself.
//
// Shrink: a wavefront is split into four 16-lane DPP rows.  Each 16-lane row reads
// 256 contiguous bytes (two 128-byte lines) of one rank row per load, rank rows are
// dealt round-robin to the four lane rows, and wavefronts split the Hin columns.  The
// per-lane partial dot products are reduced with four DPP adds inside the 16-lane row
// and across wavefronts through LDS.
// Expand: every lane owns 8 contiguous output columns, so a wavefront reads 1 KiB
// contiguous from each B rank row and writes y with 16-byte stores.  With PF the first B rows
// and the y rows of a lane's first output chunk are requested before the reduction, into the
// registers the A rows have just vacated, so the expand does not start on a cold pipe (measured:
// up to 20 % at four tokens per item and rank 64, nothing or a small loss at one or two tokens).
//
// Replaces punica.ops.add_lora_bgmv as called from lightllm/models/lora_gpu.py:138,150,162.
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

__device__ __forceinline__ int pool_row(const int32_t *__restrict__ tbl, long long dense_stride, int adapter, int j,
                                        const PoolView &pv, long long n_rows)
{
    long long row;
    if (tbl) {
        int pg = tbl[(long long)adapter * pv.max_pages + (j >> pv.page_shift)];
        row = pg < 0 ? -1 : (((long long)pg << pv.page_shift) + (j & ((1 << pv.page_shift) - 1)));
    } else {
        row = (long long)adapter * dense_stride + j;
    }
    return (row < 0 || row >= n_rows) ? -1 : (int)row;
}

template <int DT, int G, int RMAX, int NT, bool BT, bool WORK, bool PF>
__global__ __launch_bounds__(NT) void bgmv_kernel(const BgmvArgs p)
{
    constexpr int NW = NT / 64;
    constexpr int RPG = RMAX / 4;                               // rank rows per 16-lane row
    constexpr int UB = 32 / (RPG + G);                          // ~128 VGPRs of loads in flight
    constexpr int U = UB >= 4 ? 4 : (UB >= 2 ? 2 : 1);          // column steps kept in flight
    constexpr int EB = RMAX < 16 ? RMAX : 16;                   // B rank rows in flight per lane
    __shared__ float s_part[NW][G][RMAX];
    __shared__ __attribute__((aligned(16))) float s_v[G][RMAX];
    __shared__ int s_arow[WORK ? 1 : RMAX];
    __shared__ int s_brow[WORK ? 1 : RMAX];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 15, rg = lane >> 4;
    const PoolView &pv = p.pool;

    int proj, ntok = 1, adapter, r;
    float scale;
    int tok[G];
    const int32_t *__restrict__ rows = nullptr;                 // WORK: row index of rank row j at rows[j]

    if constexpr (WORK) {
        // Records are stored in launch order: record b belongs to workgroup b of every projection.
        // The gather interleaves consecutive chunks over the 8 XCDs (workgroups are dealt to XCDs
        // round-robin by id), so the chunks of one hot adapter share one XCD's L2.
        const int b = blockIdx.x % p.items_cap;
        proj = blockIdx.x / p.items_cap;
        const int32_t *__restrict__ rec = p.work + (size_t)b * WORK_WORDS;
        ntok = rec[0];
        if (ntok <= 0) return;
        ntok = ntok < G ? ntok : G;
        adapter = rec[1];
        r = rec[2];
        scale = __builtin_bit_cast(float, rec[3]);
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int t = k < ntok ? rec[4 + k] : -1;
            tok[k] = (t >= 0 && t < p.T) ? t : -1;
        }
        rows = rec + WORK_ROWS_AT;
    } else {
        const int item = blockIdx.x % p.T;
        proj = blockIdx.x / p.T;
        tok[0] = item;
#pragma unroll
        for (int k = 1; k < G; k++) tok[k] = -1;
        if (p.tok_adapter) {
            // int32 ids: any negative id and any id beyond the pool mean "no adapter" (the row is
            // defined: kept when accumulating, zeros otherwise), as the work-record path treats them
            adapter = p.tok_adapter[item];
            if (adapter < 0 || adapter >= pv.n_adapters) adapter = -1;
        } else {
            // int64 ids of the reference-layout call: a bad index leaves the row untouched (-2)
            const long long a64 = p.tok_adapter64[item];
            adapter = (a64 < 0 || a64 >= pv.n_adapters) ? -2 : (int)a64;
        }
        r = 0;
        scale = 0.f;
        if (adapter >= 0) {
            r = pv.rank ? pv.rank[adapter] : pv.uniform_rank;
            scale = pv.scaling ? pv.scaling[adapter] : pv.uniform_scale;
            if (pv.a_tbl || pv.b_tbl) {
                const int cap = pv.max_pages << pv.page_shift;
                r = r > cap ? cap : r;
            }
        }
    }
    r = r < 0 ? 0 : (r > RMAX ? RMAX : r);

    const int hin = p.hin[proj], hout = p.hout[proj];
    const uint16_t *__restrict__ x = static_cast<const uint16_t *>(p.x[proj]);
    uint16_t *__restrict__ y = static_cast<uint16_t *>(p.y[proj]);
    const uint16_t *__restrict__ arows = static_cast<const uint16_t *>(p.a_rows[proj]);
    const uint16_t *__restrict__ brows = static_cast<const uint16_t *>(p.b_rows[proj]);
    const int ncc_out = hout >> 3;

    if (adapter < 0) {
        // No adapter: y = delta mode must still define the row (zeros).  The reference-layout
        // call (tok_adapter64) leaves rows with a bad index untouched.
        if (!p.accumulate && adapter == -1) {
#pragma unroll
            for (int k = 0; k < G; k++)
                if (tok[k] >= 0)
                    for (int cc = tid; cc < ncc_out; cc += NT) stg16(y + (size_t)tok[k] * hout + (size_t)cc * 8, zero16());
        }
        return;
    }

    if constexpr (!WORK) {
        // Row index of every rank row, looked up once per work item (-1 = absent / out of bounds).
        for (int j = tid; j < RMAX; j += NT) {
            s_arow[j] = j < r ? pool_row(pv.a_tbl, pv.a_dense_stride, adapter, j, pv, pv.n_rows_a) : -1;
            if constexpr (!BT) s_brow[j] = j < r ? pool_row(pv.b_tbl, pv.b_dense_stride, adapter, j, pv, pv.n_rows_b) : -1;
        }
        __syncthreads();
    }
    // Row lookups.  Records hold -1 for every absent rank row, so record reads need no rank guard
    // and are issued as plain (batched) loads.
    auto a_row = [&](int j) -> int {
        if constexpr (WORK) { const int row = rows[j]; return (row >= 0 && row < pv.n_rows_a) ? row : -1; }
        else return s_arow[j];
    };
    auto b_rows_of = [&](int j0, int (&out)[EB]) {     // rows of rank rows j0 .. j0+EB-1 (wavefront-uniform)
        if constexpr (WORK) {
            if constexpr (EB % 4 == 0) {
                const int4 *q = reinterpret_cast<const int4 *>(rows + j0);
#pragma unroll
                for (int m = 0; m < EB / 4; m++) {
                    const int4 v = q[m];
                    out[4 * m] = v.x; out[4 * m + 1] = v.y; out[4 * m + 2] = v.z; out[4 * m + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int jj = 0; jj < EB; jj++) out[jj] = rows[j0 + jj];
            }
#pragma unroll
            for (int jj = 0; jj < EB; jj++) out[jj] = (out[jj] >= 0 && out[jj] < pv.n_rows_b) ? out[jj] : -1;
        } else {
#pragma unroll
            for (int jj = 0; jj < EB; jj++) out[jj] = __builtin_amdgcn_readfirstlane(s_brow[j0 + jj]);
        }
    };

    // ---------------------------------------------------------------- shrink
    // Loads are unconditional: an absent rank row reads row 0 of the slab and a token slot
    // beyond ntok reads token 0 (both discarded below), a column chunk past the end of the
    // row re-reads the last chunk with x forced to zero.
    const int ncc_in = hin >> 3;
    const int cpw = ((ncc_in + NW * 16 - 1) / (NW * 16)) * 16;   // 16-byte column chunks per wavefront
    const int n_it = cpw >> 4;
    const int c0 = wave * cpw + cl;
    const uint4 *ap[RPG];
    unsigned row_ok = 0;
#pragma unroll
    for (int i = 0; i < RPG; i++) {
        const int row = a_row(rg + 4 * i);
        row_ok |= (row >= 0 ? 1u : 0u) << i;
        ap[i] = reinterpret_cast<const uint4 *>(arows + (size_t)(row >= 0 ? row : 0) * hin);
    }
    const uint4 *xp[G];
#pragma unroll
    for (int k = 0; k < G; k++) xp[k] = reinterpret_cast<const uint4 *>(x + (size_t)(tok[k] >= 0 ? tok[k] : 0) * hin);
    float acc[G][RPG];
#pragma unroll
    for (int k = 0; k < G; k++)
#pragma unroll
        for (int i = 0; i < RPG; i++) acc[k][i] = 0.f;

#pragma unroll 1
    for (int it0 = 0; it0 < n_it; it0 += U) {
        uint4 xv[G][U];
        uint4 av[RPG][U];
        bool cv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int c = c0 + (it0 + u) * 16;
            cv[u] = (it0 + u) < n_it && c < ncc_in;
            const int cs = c < ncc_in ? c : ncc_in - 1;
#pragma unroll
            for (int k = 0; k < G; k++) xv[k][u] = ldg16_stream(xp[k] + cs);
#pragma unroll
            for (int i = 0; i < RPG; i++) av[i][u] = ldg16_stream(ap[i] + cs);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int k = 0; k < G; k++) {
                xv[k][u].x = cv[u] ? xv[k][u].x : 0u; xv[k][u].y = cv[u] ? xv[k][u].y : 0u;
                xv[k][u].z = cv[u] ? xv[k][u].z : 0u; xv[k][u].w = cv[u] ? xv[k][u].w : 0u;
            }
#pragma unroll
            for (int i = 0; i < RPG; i++)
#pragma unroll
                for (int k = 0; k < G; k++) acc[k][i] = dot8<DT>(av[i][u], xv[k][u], acc[k][i]);
        }
    }

    // First expand step requested now: its latency runs under the reduction and the two barriers.
    uint4 bpre[PF ? EB : 1];
    uint4 ypre[PF ? G : 1];
    if constexpr (PF) {
        if (tid < ncc_out) {
            int br[EB];
            b_rows_of(0, br);
#pragma unroll
            for (int jj = 0; jj < EB; jj++)
                bpre[jj] = br[jj] >= 0 ? ldg16_stream(brows + (size_t)br[jj] * hout + (size_t)tid * 8) : zero16();
#pragma unroll
            for (int k = 0; k < G; k++)
                ypre[k] = (p.accumulate && tok[k] >= 0) ? ldg16_stream(y + (size_t)tok[k] * hout + (size_t)tid * 8) : zero16();
        }
    }

#pragma unroll
    for (int k = 0; k < G; k++)
#pragma unroll
        for (int i = 0; i < RPG; i++) {
            const float a = ((row_ok >> i) & 1u) ? acc[k][i] : 0.f;
            const float s = row16_sum(a);
            if (cl == 0) s_part[wave][k][rg + 4 * i] = s;
        }
    __syncthreads();
    for (int e = tid; e < G * RMAX; e += NT) {
        const int k = e / RMAX, j = e - k * RMAX;
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < NW; wv++) s += s_part[wv][k][j];
        s_v[k][j] = j < r ? s * scale : 0.f;
    }
    __syncthreads();

    // ---------------------------------------------------------------- expand
    if constexpr (!BT) {
#pragma unroll 1
        for (int cc = tid; cc < ncc_out; cc += NT) {
            const bool pre = PF && cc == tid;            // this step's first rows and y are already in registers
            float o[G][8];
#pragma unroll
            for (int k = 0; k < G; k++) {
                if (p.accumulate && tok[k] >= 0) {
                    uint4 yv;
                    if (pre) yv = ypre[k]; else yv = ldg16_stream(y + (size_t)tok[k] * hout + (size_t)cc * 8);
                    unpack8<DT>(yv, o[k]);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) o[k][e] = 0.f;
                }
            }
#pragma unroll 1
            for (int j0 = 0; j0 < r; j0 += EB) {
                uint4 bv[EB];
                if (pre && j0 == 0) {
#pragma unroll
                    for (int jj = 0; jj < EB; jj++) bv[jj] = bpre[jj];
                } else {
                    int br[EB];
                    b_rows_of(j0, br);
#pragma unroll
                    for (int jj = 0; jj < EB; jj++)
                        bv[jj] = br[jj] >= 0 ? ldg16_stream(brows + (size_t)br[jj] * hout + (size_t)cc * 8) : zero16();
                }
#pragma unroll
                for (int jj = 0; jj < EB; jj++) {
                    float f[8];
                    unpack8<DT>(bv[jj], f);
#pragma unroll
                    for (int k = 0; k < G; k++) {
                        const float vk = s_v[k][j0 + jj];
#pragma unroll
                        for (int e = 0; e < 8; e++) o[k][e] = fmaf(vk, f[e], o[k][e]);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < G; k++)
                if (tok[k] >= 0) stg16_stream(y + (size_t)tok[k] * hout + (size_t)cc * 8, pack8<DT>(o[k]));
        }
    } else {
        // B given as [hout, r] blocks (reference layout): output column c is the dot product
        // of v with the r contiguous values at brows + adapter * stride + c * r.
        const uint16_t *__restrict__ bt = brows + (size_t)adapter * (size_t)pv.b_dense_stride;
        if ((r & 7) == 0) {
            const int npair = hout >> 1;
            for (int cp = tid; cp < npair; cp += NT) {
                float o[G][2];
#pragma unroll
                for (int k = 0; k < G; k++) {
                    o[k][0] = 0.f; o[k][1] = 0.f;
                    if (p.accumulate && tok[k] >= 0) {
                        const uint32_t u = *reinterpret_cast<const uint32_t *>(y + (size_t)tok[k] * hout + (size_t)cp * 2);
                        o[k][0] = lo_f32<DT>(u); o[k][1] = hi_f32<DT>(u);
                    }
                }
                const uint16_t *b0 = bt + (size_t)cp * 2 * r;
#pragma unroll
                for (int j0 = 0; j0 < RMAX; j0 += 8) {
                    if (j0 < r) {
                        float f0[8], f1[8];
                        unpack8<DT>(ldg16(b0 + j0), f0);
                        unpack8<DT>(ldg16(b0 + r + j0), f1);
#pragma unroll
                        for (int k = 0; k < G; k++)
#pragma unroll
                            for (int e = 0; e < 8; e++) {
                                const float vk = s_v[k][j0 + e];
                                o[k][0] = fmaf(vk, f0[e], o[k][0]);
                                o[k][1] = fmaf(vk, f1[e], o[k][1]);
                            }
                    }
                }
#pragma unroll
                for (int k = 0; k < G; k++)
                    if (tok[k] >= 0)
                        *reinterpret_cast<uint32_t *>(y + (size_t)tok[k] * hout + (size_t)cp * 2) = pack2<DT>(o[k][0], o[k][1]);
            }
        } else {
            for (int c = tid; c < hout; c += NT) {
                float o[G];
#pragma unroll
                for (int k = 0; k < G; k++) {
                    o[k] = 0.f;
                    if (p.accumulate && tok[k] >= 0) {
                        const uint32_t u = y[(size_t)tok[k] * hout + c];
                        o[k] = lo_f32<DT>(u);
                    }
                }
                for (int j = 0; j < r; j++) {
                    const float b = lo_f32<DT>((uint32_t)bt[(size_t)c * r + j]);
#pragma unroll
                    for (int k = 0; k < G; k++) o[k] = fmaf(s_v[k][j], b, o[k]);
                }
#pragma unroll
                for (int k = 0; k < G; k++)
                    if (tok[k] >= 0) y[(size_t)tok[k] * hout + c] = (uint16_t)cvt16<DT>(o[k]);
            }
        }
    }
}

template <int DT, int G, int RMAX, bool BT, bool WORK>
static int launch_one(const BgmvArgs &a, hipStream_t s)
{
    // Work items of one or two tokens are the small-batch form: a launch of at most about one
    // workgroup per CU, bound by the chain launch -> record -> page table -> rows -> y.  Twice the
    // threads halve the shrink's load rounds and the early expand requests overlap the reduction
    // (8.5 vs 9.9 us per call at 64 tokens, 10.8 vs 13.2 us at 128, three projections).
    constexpr bool WIDE = WORK && !BT && G <= 2;
    constexpr int NT = WIDE ? 512 : 256;
    const long long per_proj = WORK ? a.items_cap : a.T;
    const long long total = (long long)a.n_proj * per_proj;
    if (total <= 0) return 0;
    if (total > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    // Early expand requests pay for their registers when a work item carries several tokens, or when
    // the launch is latency-bound anyway.
    constexpr bool PF = WORK && !BT && (G >= 4 || WIDE);
    hipLaunchKernelGGL((bgmv_kernel<DT, G, RMAX, NT, BT, WORK, PF>), dim3((unsigned)total), dim3(NT), 0, s, a);
    return (int)hipGetLastError();
}

template <int DT, int RMAX>
static int launch_work(const BgmvArgs &a, int group, hipStream_t s)
{
    switch (group) {
    case 1: return launch_one<DT, 1, RMAX, false, true>(a, s);
    case 2: return launch_one<DT, 2, RMAX, false, true>(a, s);
    case 4: return launch_one<DT, 4, RMAX, false, true>(a, s);
    case 8:
        if constexpr (RMAX <= 32) return launch_one<DT, 8, RMAX, false, true>(a, s);
        else return (int)hipErrorInvalidValue;
    default: return (int)hipErrorInvalidValue;
    }
}

template <int DT>
static int launch_dt(const BgmvArgs &a, int group, int max_rank, bool bt, hipStream_t s)
{
    if (a.work) {
        if (bt) return (int)hipErrorInvalidValue;
        if (max_rank <= 16) return launch_work<DT, 16>(a, group, s);
        if (max_rank <= 32) return launch_work<DT, 32>(a, group, s);
        return launch_work<DT, 64>(a, group, s);
    }
    if (group != 1) return (int)hipErrorInvalidValue;      // the plain form is one token per work item
    if (bt) {
        if (max_rank <= 16) return launch_one<DT, 1, 16, true, false>(a, s);
        if (max_rank <= 32) return launch_one<DT, 1, 32, true, false>(a, s);
        return launch_one<DT, 1, 64, true, false>(a, s);
    }
    if (max_rank <= 16) return launch_one<DT, 1, 16, false, false>(a, s);
    if (max_rank <= 32) return launch_one<DT, 1, 32, false, false>(a, s);
    return launch_one<DT, 1, 64, false, false>(a, s);
}

int launch_bgmv(const BgmvArgs &a, int dtype, int group, int max_rank, bool b_transposed, hipStream_t s)
{
    if (dtype == DT_F16) return launch_dt<DT_F16>(a, group, max_rank, b_transposed, s);
    return launch_dt<DT_BF16>(a, group, max_rank, b_transposed, s);
}

}  // namespace mlora
