// BGMV decode as two launches for gfx950: a shrink launch that writes x . A as fp32 partial sums
// per slice of the Hin columns, and an expand launch that sums the slices, scales and applies B.
//
// Why two launches when one can keep the intermediate on chip: a compute unit can only keep a
// limited number of cache-line fills in flight, so the chip reaches its memory bandwidth only
// while every compute unit is pulling data.  The fused kernel's unit of work is a whole item
// (an adapter's A and B rows for one projection, hundreds of KiB) and a decode batch has about
// one item per compute unit, so a unit that gets two items finishes late and the others idle.
// Here the unit of work is a 1024- or 2048-column slice of an item (tens of KiB), there are several
// slices per compute unit and per phase, and no row is fetched by more than one workgroup.
// The price is the intermediate (T x slices x rank fp32, a few hundred KiB) going through L2.
//
// Both kernels read the work records the gather wrote (one 320-byte record per item: tokens,
// adapter, rank, scaling, the row of every rank row).  Workgroup ids are record-major: the slices
// and projections of record 0, then those of record 1, ...  Ids go to the eight XCDs round-robin,
// so the eight workgroups that run side by side read neighbouring column slices of the same rank
// rows (whole rows, back to back in DRAM) instead of the same slice of eight different adapters;
// measured against the other order (eight records, one per XCD, then their slices): the
// mixed-rank batch of 128 tokens 7 % faster, the 512-token batch 1 %, the 256-token batch equal.
// The records in use come first in the gather's order, so the empty tail costs no waiting.
//
// The kernels come in two instantiations, chosen by the host from the size of the batch (launch_sliced):
//   BIG = false, a launch of about one round of workgroups (hundreds to a few thousand slices): one workgroup
//     per (record, projection, slice) over the host's upper bound on the records, nontemporal row loads; what
//     counts is the chain of dependent loads of one workgroup;
//   BIG = true, a launch of many rounds (config 5: 8000 shrink slices): the grid covers fewer records and a
//     workgroup walks records b, b + stride, ..., a rank-32 item takes two shrink slices per workgroup, rows are
//     read with ordinary loads, the record header as constant memory; what counts is throughput.
//
// Replaces punica.ops.add_lora_bgmv as called from lightllm/models/lora_gpu.py:138,150,162.
#include <type_traits>
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {


// How a launch reads the adapter rows, chosen by the host from the size of the batch:
//   HOT = false: the launch is about one round of workgroups, all items of an adapter run at the same time and the
//     rows pass through L2 once: nontemporal loads, which do not displace records and sums;
//   HOT = true: a launch of many rounds of workgroups; the later items of a much-used adapter find its rows in L2
//     only if they are kept: ordinary loads (nontemporal ones measured 3 % slower in the shrink and 10 % in the
//     expand of the 512-token batch; choosing per item, by whether the neighbouring records name the same adapter,
//     measured slower than either).
template <bool HOT>
__device__ __forceinline__ uint4 ld_rows(const void *p) { if constexpr (HOT) return ldg16(p); else return ldg16_stream(p); }

// A work record as the kernels read it.  In a one-round launch (no loop over records) an ordinary pointer: the
// compiler already fetches the header with scalar loads and the allocation it reaches with that is the measured
// best; in a launch of many rounds the record is read as constant memory, which keeps the header loads scalar
// inside the loop over records.
template <bool BIG> struct RecPtr { typedef const int32_t *__restrict__ type; };
template <> struct RecPtr<true> { typedef const_i32_ptr type; };
template <bool BIG>
__device__ __forceinline__ typename RecPtr<BIG>::type record_at(const int32_t *work, int b)
{
    if constexpr (BIG) return as_const(work + (size_t)b * WORK_WORDS);
    else return work + (size_t)b * WORK_WORDS;
}

struct ItemId { int b, q; };

__device__ __forceinline__ ItemId split_id(unsigned id, int nq)
{
    ItemId r;
    r.b = (int)(id / (unsigned)nq);
    r.q = (int)(id - (unsigned)r.b * (unsigned)nq);
    return r;
}

// Slices of the launch's width (Slices<RMAX>::KSC) that one shrink workgroup takes, by the rank bucket of
// its item (more than 32, 17..32, 9..16, at most 8 rank rows): the bytes of a workgroup grow with
// rank x width, so an item of low rank in a launch sized for rank 64 takes wider slices.
template <int RMAX, bool BIG> struct SliceFactor;
template <bool BIG> struct SliceFactor<16, BIG> { static constexpr int F16 = 1, F8 = 1, F4 = 1, F2 = 1; };
template <bool BIG> struct SliceFactor<32, BIG> { static constexpr int F16 = 1, F8 = BIG ? 2 : 1, F4 = 2, F2 = 4; };
template <bool BIG> struct SliceFactor<64, BIG> { static constexpr int F16 = 1, F8 = 1, F4 = 2, F2 = 4; };
template <int RMAX, bool BIG>
__device__ __forceinline__ int slice_factor(int r)
{
    using SF = SliceFactor<RMAX, BIG>;
    return r > 32 ? SF::F16 : (r > 16 ? SF::F8 : (r > 8 ? SF::F4 : SF::F2));
}

// Shrink of one (item, projection, column slice) over the first 4 * NR rank rows (NR per 16-lane
// row).  The caller picks the smallest NR that covers the item's rank, so an adapter of rank 8 in a
// pool that goes up to rank 64 issues loads for 8 rows, not 64.
template <int DT, int G, int RMAX, int KSC, int NR, bool HOT, class RowsPtr>
__device__ __forceinline__ void shrink_rows(const BgmvArgs &p, RowsPtr rows, const int (&tok)[G],
                                            int r, int proj, int ks, int slot, float (&s_part)[4][G][RMAX])
{
    constexpr int NW = 4;
    constexpr int STEPS = KSC / 64;                             // 16-chunk steps per wavefront
    constexpr int UW = (NR + G) <= 12 ? 2 : 1;
    constexpr int U = UW < STEPS ? UW : STEPS;                  // column steps kept in flight
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 15, rg = lane >> 4;
    const PoolView &pv = p.pool;
    const int hin = p.hin[proj];
    const int ncc_in = hin >> 3;
    const int kc0 = ks * KSC;
    const uint16_t *__restrict__ x = static_cast<const uint16_t *>(p.x[proj]);
    const uint16_t *__restrict__ arows = static_cast<const uint16_t *>(p.a_rows[proj]);

    // Loads are unconditional: an absent rank row reads row 0 of the slab and a token slot beyond
    // ntok reads token 0 (both discarded below).  Each wavefront covers a quarter of the slice in steps
    // of 16 chunks per 16-lane row.  A slice that lies inside the row (all but a projection's last one)
    // is read at fixed distances from one address per row, so the loads need no address registers of
    // their own; the last, partial slice re-reads the row's last chunk for chunks past the end, with x
    // forced to zero.
    const int c_first = kc0 + wave * (STEPS * 16) + cl;
    const bool whole = kc0 + KSC <= ncc_in;                     // uniform over the workgroup
    const uint4 *ap[NR];
    unsigned row_ok = 0;
#pragma unroll
    for (int i = 0; i < NR; i++) {
        int row = rows[rg + 4 * i];
        row = (row >= 0 && row < pv.n_rows_a) ? row : -1;
        row_ok |= (row >= 0 ? 1u : 0u) << i;
        ap[i] = reinterpret_cast<const uint4 *>(arows + (size_t)(row >= 0 ? row : 0) * hin) + (whole ? c_first : 0);
    }
    const uint4 *xp[G];
#pragma unroll
    for (int k = 0; k < G; k++)
        xp[k] = reinterpret_cast<const uint4 *>(x + (size_t)(tok[k] >= 0 ? tok[k] : 0) * hin) + (whole ? c_first : 0);
    float acc[G][NR];
#pragma unroll
    for (int k = 0; k < G; k++)
#pragma unroll
        for (int i = 0; i < NR; i++) acc[k][i] = 0.f;

    if (whole) {
#pragma unroll
        for (int it0 = 0; it0 < STEPS; it0 += U) {
            uint4 xv[G][U];
            uint4 av[NR][U];
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int k = 0; k < G; k++) xv[k][u] = ldg16_stream(xp[k] + (it0 + u) * 16);
#pragma unroll
                for (int i = 0; i < NR; i++) av[i][u] = ld_rows<HOT>(ap[i] + (it0 + u) * 16);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int i = 0; i < NR; i++)
#pragma unroll
                    for (int k = 0; k < G; k++) acc[k][i] = dot8<DT>(av[i][u], xv[k][u], acc[k][i]);
        }
    } else {
#pragma unroll 1
        for (int it = 0; it < STEPS; it++) {
            const int c = c_first + it * 16;
            const bool cv = c < ncc_in;
            const int cs = cv ? c : ncc_in - 1;
            uint4 xv[G];
            uint4 av[NR];
#pragma unroll
            for (int k = 0; k < G; k++) xv[k] = ldg16_stream(xp[k] + cs);
#pragma unroll
            for (int i = 0; i < NR; i++) av[i] = ld_rows<HOT>(ap[i] + cs);
#pragma unroll
            for (int k = 0; k < G; k++) {
                xv[k].x = cv ? xv[k].x : 0u; xv[k].y = cv ? xv[k].y : 0u;
                xv[k].z = cv ? xv[k].z : 0u; xv[k].w = cv ? xv[k].w : 0u;
            }
#pragma unroll
            for (int i = 0; i < NR; i++)
#pragma unroll
                for (int k = 0; k < G; k++) acc[k][i] = dot8<DT>(av[i], xv[k], acc[k][i]);
        }
    }

#pragma unroll
    for (int k = 0; k < G; k++)
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const float a = ((row_ok >> i) & 1u) ? acc[k][i] : 0.f;
            const float s = row16_sum(a);
            if (cl == 0) s_part[wave][k][rg + 4 * i] = s;
        }
    __syncthreads();
    for (int e = tid; e < G * 4 * NR; e += 256) {
        const int k = e / (4 * NR), j = e - k * (4 * NR);
        if (j < r && tok[k] >= 0) {
            float s = 0.f;
#pragma unroll
            for (int wv = 0; wv < NW; wv++) s += s_part[wv][k][j];
            p.vws[(((size_t)proj * p.T + tok[k]) * p.ks_max + slot) * RMAX + j] = s;
        }
    }
}

template <int DT, int G, int RMAX, int KSC, bool BIG>
__global__ __launch_bounds__(256) void bgmv_shrink_kernel(const BgmvArgs p)
{
    __shared__ float s_part[4][G][RMAX];

    // workgroup -> (record, projection, slice): only the slices a projection has are numbered
    const ItemId id = split_id(blockIdx.x, p.sh_end[p.n_proj - 1]);
    int proj = 0;
    while (proj + 1 < p.n_proj && id.q >= p.sh_end[proj]) proj++;
    const int ks = id.q - (proj ? p.sh_end[proj - 1] : 0);
    // A workgroup serves records id.b, id.b + stride, ...: the launch covers `rec_stride` records, not the
    // host's upper bound on them (the records in use of one XCD residue are a prefix, so the first empty one ends
    // the walk).  Most batches need one pass; what a grid over the whole bound would spend on dispatching
    // workgroups of empty records is saved.
    int b = id.b;
    do {
        const typename RecPtr<BIG>::type rec = record_at<BIG>(p.work, b);
        int ntok = rec[0];
        if (ntok <= 0) break;
        ntok = ntok < G ? ntok : G;
        const int adapter = rec[1];
        if (adapter < 0) continue;
        int r = rec[2];
        r = r < 0 ? 0 : (r > RMAX ? RMAX : r);
        int tok[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int t = k < ntok ? rec[4 + k] : -1;
            tok[k] = (t >= 0 && t < p.T) ? t : -1;
        }
        const typename RecPtr<BIG>::type rows = rec + WORK_ROWS_AT;

        // r is uniform over the workgroup: a scalar branch, no divergence.  An item of a lower rank bucket
        // takes F consecutive slices in one workgroup (the others of the F skip it) and stores its sums
        // in the slot of the first.
        auto go = [&](auto nr_tag, auto f_tag) {
            constexpr int NR = decltype(nr_tag)::value, F = decltype(f_tag)::value;
            if (ks % F) return;
            shrink_rows<DT, G, RMAX, KSC * F, NR, BIG>(p, rows, tok, r, proj, ks / F, ks, s_part);
            if constexpr (BIG) __syncthreads();                 // s_part is reused by the next record
        };
        using SF = SliceFactor<RMAX, BIG>;
        if constexpr (RMAX >= 64) {
            if (r > 32) { go(std::integral_constant<int, 16>{}, std::integral_constant<int, SF::F16>{}); continue; }
        }
        if constexpr (RMAX >= 32) {
            if (r > 16) { go(std::integral_constant<int, 8>{}, std::integral_constant<int, SF::F8>{}); continue; }
        }
        if (r > 8) { go(std::integral_constant<int, 4>{}, std::integral_constant<int, SF::F4>{}); continue; }
        go(std::integral_constant<int, 2>{}, std::integral_constant<int, SF::F2>{});
    } while (BIG && (b += p.rec_stride_sh) < p.items_cap);
}

template <int DT, int G, int RMAX, int KSC, int NTE, bool BIG>
__global__ __launch_bounds__(NTE) void bgmv_expand_kernel(const BgmvArgs p)
{
    constexpr int NT = NTE;                                    // one 16-byte chunk of the slice per thread
    constexpr int EB = RMAX < 8 ? RMAX : 8;                     // B rank rows in flight per lane
    __shared__ __attribute__((aligned(16))) float s_v[G][RMAX];

    const int tid = threadIdx.x;
    const PoolView &pv = p.pool;

    const ItemId id = split_id(blockIdx.x, p.ex_end[p.n_proj - 1]);
    int proj = 0;
    while (proj + 1 < p.n_proj && id.q >= p.ex_end[proj]) proj++;
    const int cs = id.q - (proj ? p.ex_end[proj - 1] : 0);
    const int hout = p.hout[proj];
    const int ncc_out = hout >> 3;
    const int cc = cs * NTE + tid;
    const bool active = cc < ncc_out;
    uint16_t *__restrict__ y = static_cast<uint16_t *>(p.y[proj]);
    const uint16_t *__restrict__ brows = static_cast<const uint16_t *>(p.b_rows[proj]);
    const unsigned voff = (unsigned)(active ? cc : 0) * 16u;
    const int n_ks = ((p.hin[proj] >> 3) + KSC - 1) / KSC;

    // records id.b, id.b + stride, ... (see the shrink kernel)
    int b = id.b;
    do {
        const typename RecPtr<BIG>::type rec = record_at<BIG>(p.work, b);
        int ntok = rec[0];
        if (ntok <= 0) break;
        ntok = ntok < G ? ntok : G;
        const int adapter = rec[1];
        int r = rec[2];
        r = r < 0 ? 0 : (r > RMAX ? RMAX : r);
        const float scale = __builtin_bit_cast(float, rec[3]);
        int tok[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int t = k < ntok ? rec[4 + k] : -1;
            tok[k] = (t >= 0 && t < p.T) ? t : -1;
        }
        const typename RecPtr<BIG>::type rows = rec + WORK_ROWS_AT;

        if (adapter < 0) {
            if (!p.accumulate && active) {
#pragma unroll
                for (int k = 0; k < G; k++)
                    if (tok[k] >= 0) stg16(y + (size_t)tok[k] * hout + (size_t)cc * 8, zero16());
            }
            continue;
        }

        auto b_rows_of = [&](int j0, int (&out)[EB]) {              // rows of rank rows j0 .. j0+EB-1
            if constexpr (!BIG && EB % 4 == 0) {
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
        };

        // A rank row's address is the same for the whole workgroup (scalar registers) and a lane adds its column
        // offset; an absent row reads row 0 and is zeroed afterwards, so a batch of loads is issued without a branch.
        auto load_b = [&](int j0, uint4 (&out)[EB]) {
            int br[EB];
            b_rows_of(j0, br);
            if constexpr (!BIG) {
#pragma unroll
                for (int jj = 0; jj < EB; jj++)
                    out[jj] = br[jj] >= 0 ? ldg16_stream(brows + (size_t)br[jj] * hout + (size_t)cc * 8) : zero16();
                return;
            }
#pragma unroll
            for (int jj = 0; jj < EB; jj++) {
                const int row = __builtin_amdgcn_readfirstlane(br[jj]);
                const char *rp = reinterpret_cast<const char *>(brows) + (size_t)(row >= 0 ? row : 0) * (size_t)hout * 2u;
                out[jj] = ldg16(rp + voff);
                if (row < 0) out[jj] = zero16();
            }
        };
        // Everything the first step needs is requested before the partial sums are fetched.
        uint4 bv[EB];
        uint4 yv[G];
        if (active) {
            load_b(0, bv);
#pragma unroll
            for (int k = 0; k < G; k++)
                yv[k] = (p.accumulate && tok[k] >= 0) ? ldg16_stream(y + (size_t)tok[k] * hout + (size_t)cc * 8) : zero16();
        }

        // v = scaling * (sum of the slices' partial sums), slices added in ascending order.
        const int kstep = slice_factor<RMAX, BIG>(r);                   // the shrink filled every kstep-th slot
        for (int e = tid; e < G * RMAX; e += NT) {
            const int k = e / RMAX, j = e - k * RMAX;
            float s = 0.f;
            if (j < r && tok[k] >= 0) {
                // eight slices' sums are requested at once (one round trip instead of one per slice) and added in
                // ascending slice order
                const float *src = p.vws + (((size_t)proj * p.T + tok[k]) * p.ks_max) * RMAX + j;
                for (int ks0 = 0; ks0 < n_ks; ks0 += 8 * kstep) {
                    float t[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const int ks = ks0 + u * kstep;
                        t[u] = ks < n_ks ? src[(size_t)ks * RMAX] : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < 8; u++) s += t[u];
                }
            }
            s_v[k][j] = s * scale;
        }
        __syncthreads();
        if (active) {
            float o[G][8];
#pragma unroll
            for (int k = 0; k < G; k++) unpack8<DT>(yv[k], o[k]);
#pragma unroll 1
            for (int j0 = 0; j0 < r; j0 += EB) {
                if (j0 > 0) load_b(j0, bv);
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
        if constexpr (BIG) __syncthreads();                     // s_v is reused by the next record
    } while (BIG && (b += p.rec_stride_ex) < p.items_cap);
}

// Slice sizes per rank bucket, in 16-byte chunks (8 columns): the bytes of a shrink workgroup grow
// with rank x slice width, so wider ranks take narrower slices (measured over 64 / 128 / 256 chunks
// on rank-16, rank-32, rank-64 and mixed-rank batches).  Expand slices: 2048 columns (256 threads) at
// rank <= 16, 1024 columns (128 threads) above: with the record-major order of the workgroups the
// narrower slices measured 2 % faster on the 512-token rank-32 batch and 1 % on the mixed-rank one
// (512 columns the same, and 1024 at rank 16 2 % slower).
template <int RMAX> struct Slices;
template <> struct Slices<16> { static constexpr int KSC = 256, NTE = 256; };
template <> struct Slices<32> { static constexpr int KSC = 128, NTE = 128; };
template <> struct Slices<64> { static constexpr int KSC = 128, NTE = 128; };
// Sum over each aligned group of LPC lanes (1, 2, 4 or 8); every lane of the group gets the sum.
template <int LPC>
__device__ __forceinline__ float group_sum(float v)
{
    if constexpr (LPC >= 2) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
    if constexpr (LPC >= 4) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
    if constexpr (LPC >= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));  // row_half_mirror
    return v;
}

// Expand on the reference's layout: B is given as one [hout, R] block per adapter and layer (wb_T_all of
// lightllm/models/lora_gpu.py:34,37,40), i.e. the R values of an output column lie next to each other and the
// columns of a slice form one contiguous run.  A workgroup walks its 2048-column slice in sub-tiles of 256
// columns: the sub-tile's run of 256 * R values is read with fully coalesced 16-byte loads (chunk q = 256 i + t
// holds 8 ranks of column q / (R / 8)), every lane multiplies its 8 ranks with the matching 8 intermediates of
// each token, the R / 8 lanes of a column are added with DPP moves, and the sums pass through LDS so that y is
// updated with 16-byte, row-contiguous accesses.  The next sub-tile's loads are in flight during the arithmetic.
template <int DT, int G, int R, int KSC>
__global__ __launch_bounds__(256) void bgmv_expand_bt_kernel(const BgmvArgs p)
{
    constexpr int RMAX = R <= 16 ? 16 : (R <= 32 ? 32 : 64);   // rank stride of the shrink's partial sums
    constexpr int LPC = R / 8;                                  // lanes per column
    constexpr int CPP = 256 / LPC;                              // columns per pass of 256 chunks
    constexpr int SUB = 256;                                    // columns per sub-tile
    constexpr int SLICE = 2048;                                 // columns per workgroup
    __shared__ __attribute__((aligned(16))) float s_v[G][RMAX];
    __shared__ __attribute__((aligned(16))) float s_out[2][G][SUB];

    const int tid = threadIdx.x;
    const ItemId id = split_id(blockIdx.x, p.ex_end[p.n_proj - 1]);
    int proj = 0;
    while (proj + 1 < p.n_proj && id.q >= p.ex_end[proj]) proj++;
    const int cs = id.q - (proj ? p.ex_end[proj - 1] : 0);
    const int hout = p.hout[proj];
    uint16_t *__restrict__ y = static_cast<uint16_t *>(p.y[proj]);
    const int col_begin = cs * SLICE;
    const int col_end = col_begin + SLICE < hout ? col_begin + SLICE : hout;
    // y rows are handled by the first G * 32 threads: thread t -> token t / 32, 8 columns from (t % 32) * 8 of the sub-tile
    const int yk = tid >> 5, yc = (tid & 31) * 8;
    const int part = tid % LPC;                                 // which 8 ranks of a column this lane multiplies
    const int n_ks = ((p.hin[proj] >> 3) + KSC - 1) / KSC;

    const int b = id.b;
    do {
        const int32_t *__restrict__ rec = p.work + (size_t)b * WORK_WORDS;
        int ntok = rec[0];
        if (ntok <= 0) break;
        ntok = ntok < G ? ntok : G;
        const int adapter = rec[1];
        int tok[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int t = k < ntok ? rec[4 + k] : -1;
            tok[k] = (t >= 0 && t < p.T) ? t : -1;
        }
        int ytok = -1;
#pragma unroll
        for (int k = 0; k < G; k++) ytok = yk == k ? tok[k] : ytok;

        if (adapter < 0 || adapter >= p.pool.n_adapters) {
            if (!p.accumulate && ytok >= 0)
                for (int c0 = col_begin; c0 < col_end; c0 += SUB)
                    if (c0 + yc < col_end) stg16(y + (size_t)ytok * hout + c0 + yc, zero16());
            continue;
        }
        const float scale = __builtin_bit_cast(float, rec[3]) * p.pool.uniform_scale;
        const uint16_t *__restrict__ bt = static_cast<const uint16_t *>(p.b_rows[proj]) +
                                          (size_t)adapter * (size_t)p.ref_layers * (size_t)hout * R;

        uint4 bv[LPC], bn[LPC];
        auto load_sub = [&](int c0, uint4 (&out)[LPC]) {
            // chunk 256 i + t of the sub-tile's run: column c0 + i * CPP + t / LPC, ranks part * 8 ..
#pragma unroll
            for (int i = 0; i < LPC; i++) {
                const int col = c0 + i * CPP + tid / LPC;
                out[i] = col < col_end ? ldg16_stream(bt + (size_t)c0 * R + ((size_t)i * 256 + tid) * 8) : zero16();
            }
        };
        load_sub(col_begin, bv);
        uint4 yv = zero16();
        if (p.accumulate && ytok >= 0 && col_begin + yc < col_end) yv = ldg16_stream(y + (size_t)ytok * hout + col_begin + yc);

        // v = scaling * (sum of the slices' partial sums), slices added in ascending order
        for (int e = tid; e < G * RMAX; e += 256) {
            const int k = e / RMAX, j = e - k * RMAX;
            float s = 0.f;
            if (j < R && tok[k] >= 0) {
                const float *src = p.vws + (((size_t)proj * p.T + tok[k]) * p.ks_max) * RMAX + j;
                for (int ks0 = 0; ks0 < n_ks; ks0 += 8) {
                    float t8[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) t8[u] = ks0 + u < n_ks ? src[(size_t)(ks0 + u) * RMAX] : 0.f;
#pragma unroll
                    for (int u = 0; u < 8; u++) s += t8[u];
                }
            }
            s_v[k][j] = s * scale;
        }
        __syncthreads();
        float vr[G][8];                                             // this lane's 8 intermediates of every token
#pragma unroll
        for (int k = 0; k < G; k++)
#pragma unroll
            for (int e = 0; e < 8; e++) vr[k][e] = s_v[k][part * 8 + e];

        int buf = 0;
#pragma unroll 1
        for (int c0 = col_begin; c0 < col_end; c0 += SUB, buf ^= 1) {
            const bool more = c0 + SUB < col_end;
            if (more) load_sub(c0 + SUB, bn);
            uint4 yn = zero16();
            if (more && p.accumulate && ytok >= 0 && c0 + SUB + yc < col_end) yn = ldg16_stream(y + (size_t)ytok * hout + c0 + SUB + yc);
#pragma unroll
            for (int i = 0; i < LPC; i++) {
                float f[8];
                unpack8<DT>(bv[i], f);
#pragma unroll
                for (int k = 0; k < G; k++) {
                    float d = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; e++) d = fmaf(vr[k][e], f[e], d);
                    d = group_sum<LPC>(d);
                    if (part == 0) s_out[buf][k][i * CPP + tid / LPC] = d;
                }
            }
            __syncthreads();                                        // also orders this buffer's reads of two steps ago before these writes
            if (ytok >= 0 && c0 + yc < col_end) {
                float o[8];
                unpack8<DT>(yv, o);                                 // zeros when not accumulating
                const float4_t d0 = *reinterpret_cast<const float4_t *>(&s_out[buf][yk][yc]);
                const float4_t d1 = *reinterpret_cast<const float4_t *>(&s_out[buf][yk][yc + 4]);
                o[0] += d0[0]; o[1] += d0[1]; o[2] += d0[2]; o[3] += d0[3];
                o[4] += d1[0]; o[5] += d1[1]; o[6] += d1[2]; o[7] += d1[3];
                stg16_stream(y + (size_t)ytok * hout + c0 + yc, pack8<DT>(o));
            }
#pragma unroll
            for (int i = 0; i < LPC; i++) bv[i] = bn[i];
            yv = yn;
        }
    } while (false);
}

// Records a launch covers (a multiple of 8, one per XCD residue): every workgroup walks records b, b + stride, ...
// The host only knows an upper bound on the records in use (items_cap: T/G full pieces plus one short piece per
// adapter present); a grid over the whole bound spends about a nanosecond per workgroup of an empty record on
// dispatch alone, which is a tenth of a launch of thousands of slices.  The stride is never below ceil(T/G)
// (that many records are in use whenever every token has an adapter entry) and large enough for the launch to
// hold a few rounds of workgroups, so that small batches keep one workgroup per record.
constexpr int GRID_TARGET = 3072;                               // (record, slice) pairs a many-round launch covers at least
template <int G>
static int record_stride(const BgmvArgs &a, int slices, bool big)
{
    if (!big) return a.items_cap;                               // about one round of workgroups: one per record
    long long want = (a.T + G - 1) / G;
    const long long fill = (GRID_TARGET + slices - 1) / slices;
    want = want > fill ? want : fill;
    want = (want + 7) / 8 * 8;
    return want < a.items_cap ? (int)want : a.items_cap;
}

template <int DT, int G, int R>
static int launch_pair_bt(const BgmvArgs &a0, hipStream_t s)
{
    BgmvArgs a = a0;
    a.rec_stride_sh = record_stride<G>(a, a.sh_end[a.n_proj - 1], false);
    a.rec_stride_ex = record_stride<G>(a, a.ex_end[a.n_proj - 1], false);
    constexpr int RMAX = R <= 16 ? 16 : (R <= 32 ? 32 : 64);
    constexpr int KSC = Slices<RMAX>::KSC;
    const long long n_sh = (long long)a.sh_end[a.n_proj - 1] * a.rec_stride_sh;
    const long long n_ex = (long long)a.ex_end[a.n_proj - 1] * a.rec_stride_ex;
    if (n_sh <= 0 || n_ex <= 0) return 0;
    if (n_sh > 0x7fffffffLL || n_ex > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((bgmv_shrink_kernel<DT, G, RMAX, KSC, false>), dim3((unsigned)n_sh), dim3(256), 0, s, a);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL((bgmv_expand_bt_kernel<DT, G, R, KSC>), dim3((unsigned)n_ex), dim3(256), 0, s, a);
    return (int)hipGetLastError();
}

template <int DT, int G>
static int launch_bt_rank(const BgmvArgs &a, int r, hipStream_t s)
{
    switch (r) {
    case 8: return launch_pair_bt<DT, G, 8>(a, s);
    case 16: return launch_pair_bt<DT, G, 16>(a, s);
    case 32: return launch_pair_bt<DT, G, 32>(a, s);
    case 64: return launch_pair_bt<DT, G, 64>(a, s);
    default: return (int)hipErrorInvalidValue;
    }
}

template <int DT>
static int launch_bt_dt(const BgmvArgs &a, int group, int r, hipStream_t s)
{
    switch (group) {
    case 1: return launch_bt_rank<DT, 1>(a, r, s);
    case 2: return launch_bt_rank<DT, 2>(a, r, s);
    case 4: return launch_bt_rank<DT, 4>(a, r, s);
    default: return (int)hipErrorInvalidValue;
    }
}

template <int DT, int G, int RMAX, int KSC, int NTE, bool BIG>
static int launch_pair(const BgmvArgs &a0, hipStream_t s)
{
    BgmvArgs a = a0;
    a.rec_stride_sh = record_stride<G>(a, a.sh_end[a.n_proj - 1], BIG);
    a.rec_stride_ex = record_stride<G>(a, a.ex_end[a.n_proj - 1], BIG);
    const long long n_sh = (long long)a.sh_end[a.n_proj - 1] * a.rec_stride_sh;
    const long long n_ex = (long long)a.ex_end[a.n_proj - 1] * a.rec_stride_ex;
    if (n_sh <= 0 || n_ex <= 0) return 0;
    if (n_sh > 0x7fffffffLL || n_ex > 0x7fffffffLL) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((bgmv_shrink_kernel<DT, G, RMAX, KSC, BIG>), dim3((unsigned)n_sh), dim3(256), 0, s, a);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL((bgmv_expand_kernel<DT, G, RMAX, KSC, NTE, BIG>), dim3((unsigned)n_ex), dim3(NTE), 0, s, a);
    return (int)hipGetLastError();
}

template <int DT, int G, int RMAX>
static int launch_sliced(const BgmvArgs &a, hipStream_t s)
{
    // Rounds of shrink workgroups the launch may need (host's upper bound on the work items, three workgroups per
    // compute unit): from about sixteen on, the items of a much-used adapter no longer run side by side.
    const long long rounds = (long long)a.sh_end[a.n_proj - 1] * a.items_cap / (3 * device_compute_units());
    if (rounds >= 16) return launch_pair<DT, G, RMAX, Slices<RMAX>::KSC, Slices<RMAX>::NTE, true>(a, s);
    return launch_pair<DT, G, RMAX, Slices<RMAX>::KSC, Slices<RMAX>::NTE, false>(a, s);
}
void bgmv_split_slices(int max_rank, int *ksc, int *nte, bool transposed_b)
{
    if (max_rank <= 16) { *ksc = Slices<16>::KSC; *nte = Slices<16>::NTE; }
    else if (max_rank <= 32) { *ksc = Slices<32>::KSC; *nte = Slices<32>::NTE; }
    else { *ksc = Slices<64>::KSC; *nte = Slices<64>::NTE; }
    if (transposed_b) *nte = 256;              // bgmv_expand_bt_kernel walks 2048-column slices at every rank
}

template <int DT, int RMAX>
static int launch_group(const BgmvArgs &a, int group, hipStream_t s)
{
    switch (group) {
    case 1: return launch_sliced<DT, 1, RMAX>(a, s);
    case 2: return launch_sliced<DT, 2, RMAX>(a, s);
    case 4: return launch_sliced<DT, 4, RMAX>(a, s);
    case 8:
        if constexpr (RMAX <= 32) return launch_sliced<DT, 8, RMAX>(a, s);
        else return (int)hipErrorInvalidValue;
    default: return (int)hipErrorInvalidValue;
    }
}
template <int DT>
static int launch_split_dt(const BgmvArgs &a, int group, int max_rank, hipStream_t s)
{
    if (max_rank <= 16) return launch_group<DT, 16>(a, group, s);
    if (max_rank <= 32) return launch_group<DT, 32>(a, group, s);
    return launch_group<DT, 64>(a, group, s);
}

int bgmv_split_rank_stride(int max_rank) { return max_rank <= 16 ? 16 : (max_rank <= 32 ? 32 : 64); }

int launch_bgmv_split(const BgmvArgs &a, int dtype, int group, int max_rank, hipStream_t s)
{
    if (!a.work || !a.vws) return (int)hipErrorInvalidValue;
    if (a.b_transposed) {
        if (dtype == DT_F16) return launch_bt_dt<DT_F16>(a, group, max_rank, s);
        return launch_bt_dt<DT_BF16>(a, group, max_rank, s);
    }
    if (dtype == DT_F16) return launch_split_dt<DT_F16>(a, group, max_rank, s);
    return launch_split_dt<DT_BF16>(a, group, max_rank, s);
}

}  // namespace mlora
