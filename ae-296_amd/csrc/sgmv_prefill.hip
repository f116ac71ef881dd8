// SGMV prefill kernels for gfx950: tokens are packed per segment (one adapter per segment)
//     y[t] (+)= s_a * (x[t] . A_a) . B_a
// computed on v_mfma_f32_16x16x32_{f16,bf16} tiles in four launches on one stream (the first can be shared by all projections and layers of a batch):
//   plan   : cuts every segment into tiles of at most 64 tokens (work list in the workspace);
//   shrink : V[split][t][0..R) = x[t, Kslice] . A_a[:, Kslice]^T   (split-K, fp32 partials);
//   reduce : sums the K splits and stores the result as a hi + lo pair of 16-bit values, so
//            the intermediate keeps fp32 accuracy through the second MFMA;
//   expand : y[t, cols] (+)= s_a * (Vhi + Vlo) . B_a[:, cols].
// Both MFMA operands of the shrink are read straight from global memory in operand layout
// (8 contiguous K values per lane).  The expand parks the B tile in LDS (rank must be the
// in-lane K dimension, the pool stores rank rows), reads it back with the transposing LDS read,
// and passes the output through a wavefront-private LDS tile so that every y access is a
// 16-byte, row-contiguous one (8-byte accesses straight from the accumulators were measured slower).
//
// Replaces torch.bmm(torch.bmm(x, A), B) at lightllm/models/lora_gpu.py:127-128,145-146,157-158.
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

// Activations and outputs pass through once: streaming (nontemporal) accesses.  A and B rows are
// re-read by every token tile of a segment and stay ordinary cached loads (measured: streaming them
// too loses what the other three gain).


constexpr int TM = 64;       // tokens per tile
constexpr int TN = 128;      // output columns per expand step
constexpr int SG_NT = 256;   // 4 wavefronts, 16 tokens each
constexpr int VSTRIDE = MAX_RANK;
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4_t lds_short4;

__device__ __forceinline__ int sg_pool_row(const int32_t *__restrict__ tbl, long long dense_stride, int adapter, int j,
                                           const PoolView &pv, long long n_rows)
{
    long long row;
    if (tbl) {
        const int pg = tbl[(long long)adapter * pv.max_pages + (j >> pv.page_shift)];
        row = pg < 0 ? -1 : (((long long)pg << pv.page_shift) + (j & ((1 << pv.page_shift) - 1)));
    } else {
        row = (long long)adapter * dense_stride + j;
    }
    return (row < 0 || row >= n_rows) ? -1 : (int)row;
}

__device__ __forceinline__ void seg_of(const SgmvArgs &p, int s, int &start, int &len, int &adapter)
{
    if (p.seg_uniform_len > 0) { start = s * p.seg_uniform_len; len = p.seg_uniform_len; adapter = s; }
    else { start = p.seg_start[s]; len = p.seg_len[s]; adapter = p.seg_adapter[s]; }
    if (start < 0 || len < 0 || start > p.T) { start = 0; len = 0; }
    if (len > p.T - start) len = p.T - start;
}

// Workgroup id -> (tile, second index) for the shrink (second = K split) and the expand (second = column
// block).  Workgroups are dealt to the 8 XCDs round-robin by id and every XCD has its own L2; tiles are
// ordered by segment, so runs of XRUN consecutive tiles mostly share one adapter.  All workgroups of a
// run that have the same second index read the same slice of A (or B): they are given ids with the same
// residue mod 8, i.e. one XCD, and the residue rotates with the second index so the XCDs stay balanced.
constexpr int XRUN = 8;
__device__ __forceinline__ bool xcd_remap(int w, int n_second, int &tile, int &second)
{
    const int r = w & 7, slot = w >> 3;
    const int i = slot % XRUN;
    second = (slot / XRUN) % n_second;
    const int j = slot / (XRUN * n_second);
    const int run = ((r - second) & 7) + 8 * j;
    tile = run * XRUN + i;
    return true;
}
__host__ __device__ inline long long xcd_grid(int max_tiles, int n_second)
{
    const long long runs = (max_tiles + XRUN - 1) / XRUN;
    return 8LL * ((runs + 7) / 8) * n_second * XRUN;
}

// Expand launches use a second order where it fits: tile-major, the column blocks of a tile next to each other, so
// that the eight workgroups running side by side (one per XCD) update one contiguous stretch of 64 y rows instead
// of the same 1 KiB column block of 64 different tiles (DRAM pages stay open: a bare read-modify-write walk over
// config 5's y is 11 % faster this way).  The blocks of a tile are numbered up to the next multiple of eight and
// rotated by the tile's run of eight, so a column block of a run stays on one XCD (its B tile is fetched into one
// L2) and the unused numbers fall on every XCD in turn.  Only where few numbers stay unused (at most an eighth):
// with 10 blocks in 16 numbers two XCDs get twice the work of the others for eight tiles at a time, the dispatcher
// hands out workgroups in order, and the launch was 9 % slower than in the order above (config 4 with 512-column
// blocks; the host therefore picks the block width so that the count fits, see tile_major in mlora_args.hpp).
__host__ __device__ inline long long expand_grid(int max_tiles, int ncb)
{
    return tile_major(ncb) ? (long long)max_tiles * ((ncb + 7) & ~7) : xcd_grid(max_tiles, ncb);
}

// ------------------------------------------------------------------ plan
__global__ __launch_bounds__(1024) void sgmv_plan_kernel(const SgmvArgs p)
{
    __shared__ int s_wave[16];
    __shared__ int s_carry;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) s_carry = 0;
    __syncthreads();
    for (int s0 = 0; s0 < p.n_seg; s0 += 1024) {
        const int s = s0 + tid;
        int start = 0, len = 0, adapter = -1;
        if (s < p.n_seg) seg_of(p, s, start, len, adapter);
        // tiles of a segment: every TM tokens from its start, or (aligned) the pieces between multiples of TM
        const int lead = p.tile_aligned ? start % TM : 0;
        const int nt = (lead + len + TM - 1) / TM;
        int v = nt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int o = __shfl_up(v, d);
            if (lane >= d) v += o;
        }
        if (lane == 63) s_wave[wave] = v;
        __syncthreads();
        int base = s_carry;
        for (int w = 0; w < wave; w++) base += s_wave[w];
        int idx = base + v - nt;
        for (int i = 0; i < nt; i++, idx++) {
            if (idx < p.max_tiles) {
                const int b = i == 0 ? start : start - lead + i * TM;
                const int e = start - lead + (i + 1) * TM < start + len ? start - lead + (i + 1) * TM : start + len;
                p.tile_seg[idx] = s;
                p.tile_tok0[idx] = b;
                p.tile_ntok[idx] = e - b;
            }
        }
        __syncthreads();
        if (tid == 1023) s_carry = base + v;
        __syncthreads();
    }
    const int n_tiles = s_carry < p.max_tiles ? s_carry : p.max_tiles;
    if (tid == 0) p.n_tiles[0] = n_tiles;
    __syncthreads();                               // tile_* written above are visible to the whole block
    // Which tokens belong to a tile at all: y = delta mode must define the rows of the others (zeros).
    for (int t = tid; t < p.T; t += 1024) p.tok_cover[t] = 0;
    __syncthreads();
    for (long long idx = tid; idx < (long long)n_tiles * TM; idx += 1024) {
        const int tl = (int)(idx / TM), k = (int)(idx - (long long)tl * TM);
        const int t = p.tile_tok0[tl] + k;
        if (k < p.tile_ntok[tl] && t >= 0 && t < p.T) p.tok_cover[t] = 1;
    }
    // Per-tile records: everything a shrink / expand workgroup needs, so that it starts from one load.
    // Headers of up to 1024 tiles at a time go through LDS (one tile per thread), then all threads
    // fill the 80-word records of that batch with one table lookup per row word.
    const PoolView &pv = p.pool;
    __shared__ int s_hdr[1024][6];
    for (int t0 = 0; t0 < n_tiles; t0 += 1024) {
        const int t = t0 + tid;
        if (t < n_tiles) {
            const int seg = p.tile_seg[t];
            int sstart, slen, adapter;
            seg_of(p, seg, sstart, slen, adapter);
            const bool real = adapter >= 0 && adapter < pv.n_adapters;
            int rk = 0, sc = 0;
            if (real) {
                rk = pv.rank ? pv.rank[adapter] : pv.uniform_rank;
                rk = rk < 0 ? 0 : (rk > MAX_RANK ? MAX_RANK : rk);
                if (pv.a_tbl) { const int cap = pv.max_pages << pv.page_shift; rk = rk > cap ? cap : rk; }
                sc = __builtin_bit_cast(int, pv.scaling ? pv.scaling[adapter] : pv.uniform_scale);
            }
            s_hdr[tid][0] = p.tile_ntok[t]; s_hdr[tid][1] = real ? adapter : -1; s_hdr[tid][2] = rk;
            s_hdr[tid][3] = sc; s_hdr[tid][4] = p.tile_tok0[t]; s_hdr[tid][5] = seg;
        }
        __syncthreads();
        const int nb = n_tiles - t0 < 1024 ? n_tiles - t0 : 1024;
        for (int idx = tid; idx < nb * TILE_WORDS; idx += 1024) {
            const int lt = idx / TILE_WORDS, w = idx - lt * TILE_WORDS;
            int val = 0;
            if (w < 6) val = s_hdr[lt][w];
            else if (w >= TILE_ROWS_AT) {
                const int j = w - TILE_ROWS_AT, adapter = s_hdr[lt][1];
                val = (adapter >= 0 && j < s_hdr[lt][2]) ? sg_pool_row(pv.a_tbl, pv.a_dense_stride, adapter, j, pv, pv.n_rows_a) : -1;
            }
            p.tile_rec[(size_t)(t0 + lt) * TILE_WORDS + w] = val;
        }
        __syncthreads();
    }
}

// ------------------------------------------------------------------ shrink
template <int DT>
__device__ __forceinline__ float4_t mfma16(const uint4 &a, const uint4 &b, float4_t c)
{
    if constexpr (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf168_t, a), __builtin_bit_cast(bf168_t, b), c, 0, 0, 0);
}

constexpr int SG_NM = 3;     // projections of one x that a shrink workgroup serves (a larger group is cut by the host)

template <int DT, int RMAX>
__global__ __launch_bounds__(SG_NT) void sgmv_shrink_kernel(const SgmvArgs p)
{
    // One workgroup: 64 tokens x RMAX ranks over one K slice, for every projection of its group (up to SG_NM
    // projections that read the same x: q, k, v; gate, up).  A stage is 128 columns: the X tile (64 rows x 256 B)
    // and one A tile per projection (RMAX rows x 256 B) are read with 16-byte loads in which every 16-lane row
    // covers 256 contiguous bytes, parked in LDS, and consumed from there as MFMA operands (8 contiguous K
    // values per lane); the X operand of a step is read from LDS once and multiplied with every projection's A.
    // The next stage's loads are in flight while this one computes.  x is fetched once per group (streaming).
    constexpr int NB = RMAX / 16;            // rank blocks of 16
    constexpr int KB = 128;                  // columns per stage
    constexpr int CPR = KB / 8;              // 16-byte chunks per row and stage
    constexpr int PITCH = KB * 2 + 32;       // LDS row pitch in bytes; the padding spreads the operand reads over the banks
                                             // (measured: no padding 2x slower, 16 bytes 6 % slower than 32, 48..144 slower again)
    constexpr int XP = TM * CPR / SG_NT;     // X loads per thread and stage (4)
    constexpr int AP = (RMAX * CPR + SG_NT - 1) / SG_NT;   // A loads per thread, projection and stage (1, 2 or 4)
    __shared__ __attribute__((aligned(16))) unsigned char s_x[TM * PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char s_a[SG_NM][RMAX * PITCH];
    int grp = 0;
    while (grp + 1 < p.n_grp && blockIdx.x >= p.grp_end[grp]) grp++;
    int tile, split;
    const int nm = p.grp_n[grp] < SG_NM ? p.grp_n[grp] : SG_NM; // projections this workgroup serves
    xcd_remap((int)(blockIdx.x - (grp ? p.grp_end[grp - 1] : 0u)), p.pr[p.grp_first[grp]].ksplit, tile, split);
    const int p0 = p.grp_first[grp];
    const SgmvProj &pj = p.pr[p0];
    if (tile >= p.n_tiles[0]) return;
    const int32_t *__restrict__ rec = p.tile_rec + (size_t)tile * TILE_WORDS;
    const int ntok = rec[0], adapter = rec[1];
    const int tok0 = rec[4];
    if (adapter < 0 || ntok <= 0 || tok0 < 0 || tok0 + ntok > p.T) return;
    const int32_t *__restrict__ rows = rec + TILE_ROWS_AT;     // -1 for every rank row that does not exist

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;

    const int hin = pj.hin;
    const uint16_t *__restrict__ x = static_cast<const uint16_t *>(pj.x);
    const int lrow = tid >> 4, lchk = tid & 15;                // this thread's row (per pass of 16) and chunk
    const uint4 *xp[XP];
#pragma unroll
    for (int q = 0; q < XP; q++) {
        int t = lrow + 16 * q;
        t = t < ntok ? t : ntok - 1;                            // tail rows repeat the last token; never stored
        xp[q] = reinterpret_cast<const uint4 *>(x + (size_t)(tok0 + t) * hin);
    }
    const uint4 *ap[SG_NM][AP];
#pragma unroll
    for (int mm = 0; mm < SG_NM; mm++) {
        const uint16_t *arows = static_cast<const uint16_t *>(p.pr[p0 + (mm < nm ? mm : 0)].a_rows);
#pragma unroll
        for (int q = 0; q < AP; q++) {
            const int j = lrow + 16 * q;
            const int row = j < RMAX ? rows[j] : -1;
            ap[mm][q] = reinterpret_cast<const uint4 *>(arows + (size_t)(row >= 0 ? row : 0) * hin);
        }
    }
    float4_t acc[SG_NM][NB];
#pragma unroll
    for (int mm = 0; mm < SG_NM; mm++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[mm][nb] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int ncc = hin >> 3;                                   // 16-byte chunks per row
    const int nstage = (ncc + CPR - 1) / CPR;
    const int per = (nstage + pj.ksplit - 1) / pj.ksplit;
    const int st0 = split * per;
    const int st1 = st0 + per < nstage ? st0 + per : nstage;
    uint4 xr[XP], ar[SG_NM][AP];
    auto load_stage = [&](int st) {
        const int c = st * CPR + lchk;
        const bool ok = c < ncc;                                // K tail: both operands become zero
        const int cs = ok ? c : ncc - 1;
#pragma unroll
        for (int q = 0; q < XP; q++) {
            xr[q] = ldg16_stream(xp[q] + cs);                   // x passes through once per group
            if (!ok) xr[q] = zero16();
        }
#pragma unroll
        for (int mm = 0; mm < SG_NM; mm++)
            if (mm < nm) {
#pragma unroll
                for (int q = 0; q < AP; q++) { ar[mm][q] = ldg16(ap[mm][q] + cs); if (!ok) ar[mm][q] = zero16(); }
            }
    };
    if (st0 < st1) load_stage(st0);
#pragma unroll 1
    for (int st = st0; st < st1; st++) {
        __syncthreads();                                        // the previous stage has been consumed
#pragma unroll
        for (int q = 0; q < XP; q++)
            *reinterpret_cast<uint4 *>(s_x + (lrow + 16 * q) * PITCH + lchk * 16) = xr[q];
#pragma unroll
        for (int mm = 0; mm < SG_NM; mm++)
            if (mm < nm) {
#pragma unroll
                for (int q = 0; q < AP; q++)
                    if (lrow + 16 * q < RMAX) *reinterpret_cast<uint4 *>(s_a[mm] + (lrow + 16 * q) * PITCH + lchk * 16) = ar[mm][q];
            }
        __syncthreads();
        if (st + 1 < st1) load_stage(st + 1);
#pragma unroll
        for (int ks = 0; ks < KB / 32; ks++) {
            const uint4 xf = *reinterpret_cast<const uint4 *>(s_x + (wave * 16 + m) * PITCH + (ks * 4 + g) * 16);
#pragma unroll
            for (int mm = 0; mm < SG_NM; mm++)
                if (mm < nm) {
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) {
                        const uint4 af = *reinterpret_cast<const uint4 *>(s_a[mm] + (nb * 16 + m) * PITCH + (ks * 4 + g) * 16);
                        acc[mm][nb] = mfma16<DT>(xf, af, acc[mm][nb]);
                    }
                }
        }
    }
    // D[token 4g+i][rank m] per 16x16 block; rank columns that do not exist are stored as zero.
#pragma unroll
    for (int mm = 0; mm < SG_NM; mm++)
        if (mm < nm) {
            float *vout = p.pr[p0 + mm].v + ((size_t)split * p.T + tok0 + wave * 16) * VSTRIDE;
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const int col = nb * 16 + m;
                const bool col_ok = rows[col] >= 0;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int trow_o = wave * 16 + 4 * g + i;
                    if (trow_o < ntok) vout[(size_t)(4 * g + i) * VSTRIDE + col] = col_ok ? acc[mm][nb][i] : 0.f;
                }
            }
        }
}

// ------------------------------------------------------------------ reduce
// vsum[t][c] = sum over K splits of the shrink partials, stored as hi + lo 16-bit halves
// (hi = round16(v), lo = round16(v - hi)) so that the expand MFMAs see the fp32 value to
// about 2^-16 relative.  One thread per (token, 8 rank columns).
template <int DT>
__device__ __forceinline__ void split_hi_lo(const float (&v)[8], uint4 &hi, uint4 &lo)
{
    uint32_t h[8], l[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        h[e] = cvt16<DT>(v[e]);
        const float back = lo_f32<DT>(h[e]);
        l[e] = cvt16<DT>(v[e] - back);
    }
    hi = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    lo = make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16));
}

template <int DT, int RMAX>
__global__ __launch_bounds__(256) void sgmv_reduce_kernel(const SgmvArgs p)
{
    constexpr int CPT = RMAX / 8;     // 8-column groups per token
    const SgmvProj &pj = p.pr[blockIdx.y];
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)p.T * CPT) return;
    const int t = (int)(idx / CPT), c0 = (int)(idx - (long long)t * CPT) * 8;
    if (p.tok_cover[t] == 0) {
        // token outside every segment: no tile touches its row.  y = delta mode defines it as zeros
        // (the CPT threads of the token share the row); accumulate mode keeps it.
        if (!p.accumulate) {
            uint16_t *__restrict__ yrow = static_cast<uint16_t *>(pj.y) + (size_t)t * pj.hout;
            for (int cc = c0 >> 3; cc < (pj.hout >> 3); cc += CPT) stg16(yrow + (size_t)cc * 8, zero16());
        }
        return;
    }
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = 0.f;
    for (int sp = 0; sp < pj.ksplit; sp++) {
        const float4_t *vp = reinterpret_cast<const float4_t *>(pj.v + ((size_t)sp * p.T + t) * VSTRIDE + c0);
        const float4_t a = vp[0], b = vp[1];
        v[0] += a[0]; v[1] += a[1]; v[2] += a[2]; v[3] += a[3];
        v[4] += b[0]; v[5] += b[1]; v[6] += b[2]; v[7] += b[3];
    }
    uint4 hi, lo;
    split_hi_lo<DT>(v, hi, lo);
    stg16(pj.vhi + (size_t)t * VSTRIDE + c0, hi);
    stg16(pj.vlo + (size_t)t * VSTRIDE + c0, lo);
}

// ------------------------------------------------------------------ expand
template <int DT, int RMAX, bool BT>
__global__ __launch_bounds__(SG_NT) void sgmv_expand_kernel(const SgmvArgs p)
{
    // One workgroup: 64 tokens (16 per wavefront) x cols_per_block output columns, 128 columns per step.
    // The B tile of a step is parked in LDS row-major and read back column-wise with the transposing LDS
    // read (the MFMA needs rank as the in-lane K dimension, the pool stores rank rows).  The 16 x 128
    // result of a wavefront goes through a wavefront-private LDS tile so that y is read and written with
    // 16-byte accesses in which a 16-lane row covers 256 contiguous bytes of one token.  Loads of y and B
    // run one step ahead of the arithmetic.
    constexpr int KP = RMAX <= 32 ? 32 : 64;   // K of the expand MFMAs (rank padded with zeros)
    constexpr int KS = KP / 32;
    constexpr int NBC = TN / 16;               // 16-column blocks per step
    constexpr int BPITCH = TN * 2 + 16;        // bytes per rank row of the LDS B tile (16-byte aligned rows)
    constexpr int OPITCH = TN + 4;             // floats per token row of the staging tile
    constexpr int TPITCH = KP * 2 + 16;        // reference layout: bytes per output column of the LDS tile (K contiguous)
    constexpr int BQ = KP * (TN / 8) / SG_NT;  // B-tile loads per thread and step (either layout: KP x TN values)
    __shared__ __attribute__((aligned(16))) unsigned char s_b[BT ? TN * TPITCH : KP * BPITCH];
    __shared__ __attribute__((aligned(16))) float s_out[SG_NT / 64][16][OPITCH];
    __shared__ int s_brow[BT ? 1 : KP];
    typedef __attribute__((address_space(3))) volatile float lds_vfloat;
    typedef __attribute__((address_space(3))) volatile float4_t lds_vfloat4;

    int proj = 0;
    while (proj + 1 < p.n_proj && blockIdx.x >= p.ex_end[proj]) proj++;
    const SgmvProj &pj = p.pr[proj];
    const int cols_per_block = pj.cols;
    int tile, colblk;
    {
        const int w = (int)(blockIdx.x - (proj ? p.ex_end[proj - 1] : 0u));
        if (tile_major(pj.ncb)) {
            const int ncb8 = (pj.ncb + 7) & ~7;
            tile = w / ncb8;
            colblk = (w - tile * ncb8 + ncb8 - ((tile >> 3) & 7)) % ncb8;
            if (colblk >= pj.ncb) return;
        } else {
            xcd_remap(w, pj.ncb, tile, colblk);
        }
    }
    if (tile >= p.n_tiles[0]) return;
    const int32_t *__restrict__ rec = p.tile_rec + (size_t)tile * TILE_WORDS;
    const int ntok = rec[0], adapter = rec[1], r = rec[2];
    const float scale = __builtin_bit_cast(float, rec[3]);
    const int tok0 = rec[4];
    const PoolView &pv = p.pool;
    if (ntok <= 0 || tok0 < 0 || tok0 + ntok > p.T) return;
    const int hout = pj.hout;
    uint16_t *__restrict__ y = static_cast<uint16_t *>(pj.y);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const int col_begin = colblk * cols_per_block;
    int col_end = col_begin + cols_per_block;
    col_end = col_end < hout ? col_end : hout;

    if (adapter < 0) {
        if (!p.accumulate) {
            // segment without adapter: y = delta means zeros
            const int cpr = (col_end - col_begin) >> 3;
            for (int e = tid; e < ntok * cpr; e += SG_NT) {
                const int t = e / cpr, c = e - t * cpr;
                stg16(y + (size_t)(tok0 + t) * hout + col_begin + c * 8, zero16());
            }
        }
        return;
    }
    if constexpr (!BT) {
        // B rows share the page table with the A rows
        for (int j = tid; j < KP; j += SG_NT) {
            const int row = j < MAX_RANK ? rec[TILE_ROWS_AT + j] : -1;
            s_brow[j] = (row >= 0 && row < pv.n_rows_b) ? row : -1;
        }
    }

    // ---- V operand: 16 tokens of this wavefront x KP ranks as a hi + lo pair of 16-bit values
    // (written by the reduce kernel); rank columns beyond the adapter's rank are zero.
    int trow = wave * 16 + m;
    trow = trow < ntok ? trow : ntok - 1;
    uint4 vhi[KS], vlo[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        const int c0 = ks * 32 + 8 * g;
        vhi[ks] = zero16(); vlo[ks] = zero16();
        if (c0 < RMAX) {
            vhi[ks] = ldg16(pj.vhi + ((size_t)(tok0 + trow) * VSTRIDE + c0));
            vlo[ks] = ldg16(pj.vlo + ((size_t)(tok0 + trow) * VSTRIDE + c0));
        }
    }
    const uint16_t *__restrict__ brows = static_cast<const uint16_t *>(pj.b_rows);
    const uint16_t *__restrict__ bt = brows + (BT ? (size_t)adapter * (size_t)pv.b_dense_stride : 0);
    __syncthreads();

    // Loads of a step (this thread's share of the B tile and of the y rows) are issued one step ahead.
    // y rows of this wavefront: lane handles (token p / 16, 16-byte chunk p % 16), p = lane + 64 q.
    uint4 y_nx[4], b_nx[BQ];
    auto prefetch = [&](int col0) {
        if (p.accumulate) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int pp = lane + 64 * q, t = pp >> 4, c = pp & 15;
                const int col = col0 + c * 8;
                const bool ok = wave * 16 + t < ntok && col < col_end;
                y_nx[q] = ok ? ldg16_stream(y + (size_t)(tok0 + wave * 16 + t) * hout + col) : zero16();
            }
        }
        if constexpr (!BT) {
#pragma unroll
            for (int q = 0; q < BQ; q++) {
                const int e = tid + q * SG_NT;
                const int j = e / (TN / 8), c = e - j * (TN / 8);
                const int row = s_brow[j];
                const int col = col0 + c * 8;
                b_nx[q] = (row >= 0 && col < col_end) ? ldg16(brows + (size_t)row * hout + col) : zero16();
            }
        } else {
            // reference layout: column c of the adapter's [hout, r] block holds its r values contiguously, so
            // the tile of TN columns is one contiguous run when r = KP; 16-byte chunk (column, 8 ranks) per load
#pragma unroll
            for (int q = 0; q < BQ; q++) {
                const int e = tid + q * SG_NT;
                const int cl = e / (KP / 8), k0 = (e - cl * (KP / 8)) * 8;
                const int col = col0 + cl;
                b_nx[q] = (col < col_end && k0 < r) ? ldg16(bt + (size_t)col * r + k0) : zero16();
            }
        }
    };
    prefetch(col_begin);
#pragma unroll 1
    for (int col0 = col_begin; col0 < col_end; col0 += TN) {
        uint4 y0[4];
#pragma unroll
        for (int q = 0; q < 4; q++) y0[q] = y_nx[q];
        if constexpr (!BT) {
            // park B[0..KP) x [col0, col0+TN) in LDS, rows beyond the rank as zeros
            __syncthreads();
#pragma unroll
            for (int q = 0; q < BQ; q++) {
                const int e = tid + q * SG_NT;
                const int j = e / (TN / 8), c = e - j * (TN / 8);
                *reinterpret_cast<uint4 *>(s_b + j * BPITCH + c * 16) = b_nx[q];
            }
            __syncthreads();
        } else {
            // park the tile column-major (K contiguous per column): exactly the in-lane order the MFMA wants
            __syncthreads();
#pragma unroll
            for (int q = 0; q < BQ; q++) {
                const int e = tid + q * SG_NT;
                const int cl = e / (KP / 8), kc = e - cl * (KP / 8);
                *reinterpret_cast<uint4 *>(s_b + cl * TPITCH + kc * 16) = b_nx[q];
            }
            __syncthreads();
        }
        if (col0 + TN < col_end) prefetch(col0 + TN);
        float4_t acc[NBC];
#pragma unroll
        for (int nb = 0; nb < NBC; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nb = 0; nb < NBC; nb++) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                uint4 bop;
                if constexpr (!BT) {
                    // lane (n = m, k group g) needs B[ks*32 + 8g + e][nb*16 + m], e < 8: a column of the row-major
                    // tile.  ds_read_b64_tr_b16 does the transpose: the 16 lanes of a group read a 4 x 16 block
                    // (lane i: row i / 4, columns 4 (i % 4) ..+3) and lane n gets the 4 rows of column n.
                    const unsigned char *src = s_b + (ks * 32 + 8 * g + (m >> 2)) * BPITCH + (nb * 16 + (m & 3) * 4) * 2;
                    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4 *)src);
                    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4 *)(src + 4 * BPITCH));
                    bop = make_uint4(__builtin_bit_cast(uint2, lo).x, __builtin_bit_cast(uint2, lo).y,
                                     __builtin_bit_cast(uint2, hi).x, __builtin_bit_cast(uint2, hi).y);
                } else {
                    bop = *reinterpret_cast<const uint4 *>(s_b + (nb * 16 + m) * TPITCH + (ks * 4 + g) * 16);
                }
                // D[token 4g+i][column m of the block]: A operand = V, B operand = B
                acc[nb] = mfma16<DT>(vhi[ks], bop, acc[nb]);
                acc[nb] = mfma16<DT>(vlo[ks], bop, acc[nb]);
            }
        }
        // ---- transpose through this wavefront's own LDS tile, then 16-byte row-contiguous y update.
        // The tile is private to the wavefront and LDS operations of one wavefront complete in order, so no
        // barrier is needed; the accesses are volatile so that the compiler keeps them in program order and
        // emits one ds_write_b32 per element (left to itself it pairs these stores into ds_write2_b32 and,
        // in the variant without the B tile, gets two of the paired offsets wrong).
        {
            lds_vfloat *so = (lds_vfloat *)&s_out[wave][4 * g][m];
#pragma unroll
            for (int nb = 0; nb < NBC; nb++)
#pragma unroll
                for (int i = 0; i < 4; i++) so[i * OPITCH + nb * 16] = acc[nb][i];
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int pp = lane + 64 * q, t = pp >> 4, c = pp & 15;
            const int col = col0 + c * 8;
            const float4_t d0 = *(lds_vfloat4 *)&s_out[wave][t][c * 8];
            const float4_t d1 = *(lds_vfloat4 *)&s_out[wave][t][c * 8 + 4];
            if (wave * 16 + t < ntok && col < col_end) {
                float o[8];
                if (p.accumulate) unpack8<DT>(y0[q], o);
                else {
#pragma unroll
                    for (int e = 0; e < 8; e++) o[e] = 0.f;
                }
                o[0] = fmaf(scale, d0[0], o[0]); o[1] = fmaf(scale, d0[1], o[1]);
                o[2] = fmaf(scale, d0[2], o[2]); o[3] = fmaf(scale, d0[3], o[3]);
                o[4] = fmaf(scale, d1[0], o[4]); o[5] = fmaf(scale, d1[1], o[5]);
                o[6] = fmaf(scale, d1[2], o[6]); o[7] = fmaf(scale, d1[3], o[7]);
                stg16_stream(y + (size_t)(tok0 + wave * 16 + t) * hout + col, pack8<DT>(o));
            }
        }
    }
}

template <int DT, int RMAX>
static int launch_rmax(const SgmvArgs &a, int phases, hipStream_t s)
{
    int rc = 0;
    if (phases & SGMV_PLAN) {
        hipLaunchKernelGGL(sgmv_plan_kernel, dim3(1), dim3(1024), 0, s, a);
        rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    if (!(phases & (SGMV_APPLY | SGMV_SHRINK))) return 0;
    // The caller has filled pr[], the shrink groups, ksplit, cols and ncb; the grid ends are set here.
    SgmvArgs g = a;
    unsigned end = 0;
    for (int q = 0; q < g.n_grp; q++) {
        end += (unsigned)xcd_grid(g.max_tiles, g.pr[g.grp_first[q]].ksplit);
        g.grp_end[q] = end;
    }
    const unsigned sgrid = end;
    end = 0;
    for (int q = 0; q < g.n_proj; q++) {
        end += (unsigned)expand_grid(g.max_tiles, g.pr[q].ncb);
        g.ex_end[q] = end;
    }
    const unsigned egrid = end;
    hipLaunchKernelGGL((sgmv_shrink_kernel<DT, RMAX>), dim3(sgrid), dim3(SG_NT), 0, s, g);
    rc = (int)hipGetLastError();
    if (rc || !(phases & SGMV_APPLY)) return rc;
    {
        const long long n = (long long)g.T * (RMAX / 8);
        hipLaunchKernelGGL((sgmv_reduce_kernel<DT, RMAX>), dim3((unsigned)((n + 255) / 256), (unsigned)g.n_proj), dim3(256), 0, s, g);
        rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    if (g.b_transposed)
        hipLaunchKernelGGL((sgmv_expand_kernel<DT, RMAX, true>), dim3(egrid), dim3(SG_NT), 0, s, g);
    else
        hipLaunchKernelGGL((sgmv_expand_kernel<DT, RMAX, false>), dim3(egrid), dim3(SG_NT), 0, s, g);
    return (int)hipGetLastError();
}

template <int DT>
static int launch_sg_dt(const SgmvArgs &a, int max_rank, int phases, hipStream_t s)
{
    if (max_rank <= 16) return launch_rmax<DT, 16>(a, phases, s);
    if (max_rank <= 32) return launch_rmax<DT, 32>(a, phases, s);
    return launch_rmax<DT, 64>(a, phases, s);
}

int launch_sgmv(const SgmvArgs &a, int dtype, int max_rank, int phases, hipStream_t s)
{
    if (dtype == DT_F16) return launch_sg_dt<DT_F16>(a, max_rank, phases, s);
    return launch_sg_dt<DT_BF16>(a, max_rank, phases, s);
}

}  // namespace mlora
