// SGMV prefill kernels for gfx950: tokens are packed per segment (one adapter per segment)
//     y[t] (+)= s_a * (x[t] . A_a) . B_a
// computed on v_mfma_f32_16x16x32_{f16,bf16} tiles in four launches on one stream:
//   plan   : cuts every segment into tiles of 64 tokens (work list in the workspace);
//   shrink : V[split][t][0..R) = x[t, Kslice] . A_a[:, Kslice]^T   (split-K, fp32 partials);
//   reduce : sums the K splits and stores the result as a hi + lo pair of 16-bit values, so
//            the intermediate keeps fp32 accuracy through the second MFMA;
//   expand : y[t, cols] (+)= s_a * (Vhi + Vlo) . B_a[:, cols].
// Both MFMA operands of the shrink are read straight from global memory in operand layout
// (8 contiguous K values per lane).  The expand stages the B tile through LDS (rank must
// be the in-lane K dimension, the pool stores rank rows) and writes y through a wave-private
// LDS transpose so that every y access is a 16-byte, row-contiguous one.
//
// Replaces torch.bmm(torch.bmm(x, A), B) at lightllm/models/lora_gpu.py:127-128,145-146,157-158.
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

constexpr int TM = 64;       // tokens per tile
constexpr int TN = 128;      // output columns per expand step
constexpr int SG_NT = 256;   // 4 wavefronts, 16 tokens each
constexpr int VSTRIDE = MAX_RANK;

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
        const int nt = (len + TM - 1) / TM;
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
                p.tile_seg[idx] = s;
                p.tile_tok0[idx] = start + i * TM;
                p.tile_ntok[idx] = len - i * TM < TM ? len - i * TM : TM;
            }
        }
        __syncthreads();
        if (tid == 1023) s_carry = base + v;
        __syncthreads();
    }
    if (tid == 0) p.n_tiles[0] = s_carry < p.max_tiles ? s_carry : p.max_tiles;
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

template <int DT, int RMAX>
__global__ __launch_bounds__(SG_NT) void sgmv_shrink_kernel(const SgmvArgs p)
{
    constexpr int NB = RMAX / 16;   // rank blocks of 16
    constexpr int KU = 4;           // K steps (of 32) in flight
    __shared__ int s_arow[RMAX];
    const int tile = blockIdx.x, split = blockIdx.y;
    if (tile >= p.n_tiles[0]) return;
    const int seg = p.tile_seg[tile];
    int sstart, slen, adapter;
    seg_of(p, seg, sstart, slen, adapter);
    const PoolView &pv = p.pool;
    if (adapter < 0 || adapter >= pv.n_adapters) return;
    const int tok0 = p.tile_tok0[tile], ntok = p.tile_ntok[tile];
    if (ntok <= 0 || tok0 < 0 || tok0 + ntok > p.T) return;
    int r = pv.rank ? pv.rank[adapter] : pv.uniform_rank;
    r = r < 0 ? 0 : (r > RMAX ? RMAX : r);
    if (pv.a_tbl) { const int cap = pv.max_pages << pv.page_shift; r = r > cap ? cap : r; }

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    for (int j = tid; j < RMAX; j += SG_NT)
        s_arow[j] = j < r ? sg_pool_row(pv.a_tbl, pv.a_dense_stride, adapter, j, pv, pv.n_rows_a) : -1;
    __syncthreads();

    const int hin = p.hin;
    const uint16_t *__restrict__ x = static_cast<const uint16_t *>(p.x);
    const uint16_t *__restrict__ arows = static_cast<const uint16_t *>(p.a_rows);
    int trow = wave * 16 + m;
    trow = trow < ntok ? trow : ntok - 1;                       // tail rows recompute the last token; never stored
    const uint4 *xp = reinterpret_cast<const uint4 *>(x + (size_t)(tok0 + trow) * hin);
    const uint4 *ap[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int row = s_arow[nb * 16 + m];
        ap[nb] = reinterpret_cast<const uint4 *>(arows + (size_t)(row >= 0 ? row : 0) * hin);
    }
    float4_t acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int ncc = hin >> 3;                                   // 16-byte chunks per row
    const int ksteps = (ncc + 3) >> 2;
    const int per = (ksteps + p.ksplit - 1) / p.ksplit;
    const int ks0 = split * per;
    const int ks1 = ks0 + per < ksteps ? ks0 + per : ksteps;
#pragma unroll 1
    for (int ks = ks0; ks < ks1; ks += KU) {
        uint4 xf[KU], af[KU][NB];
#pragma unroll
        for (int u = 0; u < KU; u++) {
            const int c = (ks + u) * 4 + g;
            const bool ok = (ks + u) < ks1 && c < ncc;
            const int cs = c < ncc ? c : ncc - 1;
            xf[u] = xp[cs];
            if (!ok) xf[u] = zero16();
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                af[u][nb] = ap[nb][cs];
                if (!ok) af[u][nb] = zero16();
            }
        }
#pragma unroll
        for (int u = 0; u < KU; u++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++) acc[nb] = mfma16<DT>(xf[u], af[u][nb], acc[nb]);
    }
    // D[token 4g+i][rank m] per 16x16 block; rank columns that do not exist are stored as zero.
    float *vout = p.v + ((size_t)split * p.T + tok0 + wave * 16) * VSTRIDE;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int col = nb * 16 + m;
        const bool col_ok = s_arow[col] >= 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int trow_o = wave * 16 + 4 * g + i;
            if (trow_o < ntok) vout[(size_t)(4 * g + i) * VSTRIDE + col] = col_ok ? acc[nb][i] : 0.f;
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
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)p.T * CPT) return;
    const int t = (int)(idx / CPT), c0 = (int)(idx - (long long)t * CPT) * 8;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = 0.f;
    for (int sp = 0; sp < p.ksplit; sp++) {
        const float4_t *vp = reinterpret_cast<const float4_t *>(p.v + ((size_t)sp * p.T + t) * VSTRIDE + c0);
        const float4_t a = vp[0], b = vp[1];
        v[0] += a[0]; v[1] += a[1]; v[2] += a[2]; v[3] += a[3];
        v[4] += b[0]; v[5] += b[1]; v[6] += b[2]; v[7] += b[3];
    }
    uint4 hi, lo;
    split_hi_lo<DT>(v, hi, lo);
    stg16(p.vhi + (size_t)t * VSTRIDE + c0, hi);
    stg16(p.vlo + (size_t)t * VSTRIDE + c0, lo);
}

// ------------------------------------------------------------------ expand
template <int DT, int RMAX, bool BT>
__global__ __launch_bounds__(SG_NT) void sgmv_expand_kernel(const SgmvArgs p, int cols_per_block)
{
    constexpr int KP = RMAX <= 32 ? 32 : 64;   // K of the expand MFMAs (rank padded with zeros)
    constexpr int KS = KP / 32;
    constexpr int NBC = TN / 16;               // 16-column blocks per step
    constexpr int BPITCH = TN * 2 + 4;         // bytes per rank row of the LDS B tile
    constexpr int OPITCH = TN + 4;             // floats per token row of the staging tile
    __shared__ __attribute__((aligned(16))) unsigned char s_b[BT ? 16 : KP * BPITCH];
    __shared__ __attribute__((aligned(16))) float s_out[SG_NT / 64][16][OPITCH];
    __shared__ int s_brow[BT ? 1 : KP];

    const int tile = blockIdx.x;
    if (tile >= p.n_tiles[0]) return;
    const int seg = p.tile_seg[tile];
    int sstart, slen, adapter;
    seg_of(p, seg, sstart, slen, adapter);
    const PoolView &pv = p.pool;
    const int tok0 = p.tile_tok0[tile], ntok = p.tile_ntok[tile];
    if (ntok <= 0 || tok0 < 0 || tok0 + ntok > p.T) return;
    const int hout = p.hout;
    uint16_t *__restrict__ y = static_cast<uint16_t *>(p.y);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const int col_begin = blockIdx.y * cols_per_block;
    int col_end = col_begin + cols_per_block;
    col_end = col_end < hout ? col_end : hout;

    if (adapter < 0 || adapter >= pv.n_adapters) {
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
    int r = pv.rank ? pv.rank[adapter] : pv.uniform_rank;
    r = r < 0 ? 0 : (r > RMAX ? RMAX : r);
    if (pv.a_tbl) { const int cap = pv.max_pages << pv.page_shift; r = r > cap ? cap : r; }
    const float scale = pv.scaling ? pv.scaling[adapter] : pv.uniform_scale;

    if constexpr (!BT) {
        for (int j = tid; j < KP; j += SG_NT)
            s_brow[j] = j < r ? sg_pool_row(pv.b_tbl, pv.b_dense_stride, adapter, j, pv, pv.n_rows_b) : -1;
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
            vhi[ks] = ldg16(p.vhi + ((size_t)(tok0 + trow) * VSTRIDE + c0));
            vlo[ks] = ldg16(p.vlo + ((size_t)(tok0 + trow) * VSTRIDE + c0));
        }
    }
    const uint16_t *__restrict__ brows = static_cast<const uint16_t *>(p.b_rows);
    const uint16_t *__restrict__ bt = brows + (BT ? (size_t)adapter * (size_t)pv.b_dense_stride : 0);
    __syncthreads();

#pragma unroll 1
    for (int col0 = col_begin; col0 < col_end; col0 += TN) {
        // y rows of this wavefront: lane handles (token p / 16, 16-byte chunk p % 16), p = lane + 64 q
        uint4 y0[4];
        if (p.accumulate) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int pp = lane + 64 * q, t = pp >> 4, c = pp & 15;
                const int col = col0 + c * 8;
                const bool ok = wave * 16 + t < ntok && col < col_end;
                y0[q] = ok ? ldg16(y + (size_t)(tok0 + wave * 16 + t) * hout + col) : zero16();
            }
        }
        if constexpr (!BT) {
            // stage B[0..KP) x [col0, col0+TN) in LDS, rows beyond the rank as zeros
            __syncthreads();
            for (int e = tid; e < KP * (TN / 8); e += SG_NT) {
                const int j = e / (TN / 8), c = e - j * (TN / 8);
                const int row = s_brow[j];
                const int col = col0 + c * 8;
                uint4 bv = zero16();
                if (row >= 0 && col < col_end) bv = ldg16(brows + (size_t)row * hout + col);
                uint32_t *dst = reinterpret_cast<uint32_t *>(s_b + j * BPITCH + c * 16);
                dst[0] = bv.x; dst[1] = bv.y; dst[2] = bv.z; dst[3] = bv.w;
            }
            __syncthreads();
        }
        float4_t acc[NBC];
#pragma unroll
        for (int nb = 0; nb < NBC; nb++) acc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nb = 0; nb < NBC; nb++) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                uint4 bop;
                if constexpr (!BT) {
                    // lane (n = m, k group g): B[ks*32 + 8g + e][col0 + nb*16 + m], e < 8
                    const unsigned char *src = s_b + (ks * 32 + 8 * g) * BPITCH + (nb * 16 + m) * 2;
                    uint32_t h[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) h[e] = *reinterpret_cast<const uint16_t *>(src + e * BPITCH);
                    bop = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
                } else {
                    const int col = col0 + nb * 16 + m;
                    const int k0 = ks * 32 + 8 * g;
                    bop = (col < col_end && k0 < r) ? ldg16(bt + (size_t)col * r + k0) : zero16();
                }
                // D[m = column][n = token] would scatter y; keep D[token][column]: A operand = V, B operand = B
                acc[nb] = mfma16<DT>(vhi[ks], bop, acc[nb]);
                acc[nb] = mfma16<DT>(vlo[ks], bop, acc[nb]);
            }
        }
        // ---- transpose through LDS (one 16 x TN tile per wavefront), then 16-byte row-contiguous y update
        {
            // volatile: one ds_write_b32 per element.  Left to itself the compiler pairs these
            // stores into ds_write2_b32 and, in the variant without the B staging tile, gets two
            // of the paired offsets wrong.
            typedef __attribute__((address_space(3))) volatile float lds_vfloat;
            lds_vfloat *so = (lds_vfloat *)&s_out[wave][4 * g][m];
#pragma unroll
            for (int nb = 0; nb < NBC; nb++)
#pragma unroll
                for (int i = 0; i < 4; i++) so[i * OPITCH + nb * 16] = acc[nb][i];
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int pp = lane + 64 * q, t = pp >> 4, c = pp & 15;
            const int col = col0 + c * 8;
            if (wave * 16 + t < ntok && col < col_end) {
                const float4_t d0 = *reinterpret_cast<const float4_t *>(&s_out[wave][t][c * 8]);
                const float4_t d1 = *reinterpret_cast<const float4_t *>(&s_out[wave][t][c * 8 + 4]);
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
                stg16(y + (size_t)(tok0 + wave * 16 + t) * hout + col, pack8<DT>(o));
            }
        }
        if constexpr (BT) __syncthreads();   // staging tile is rewritten by the next step (the B staging barrier covers !BT)
    }
}

template <int DT, int RMAX>
static int launch_rmax(const SgmvArgs &a, hipStream_t s)
{
    hipLaunchKernelGGL(sgmv_plan_kernel, dim3(1), dim3(1024), 0, s, a);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL((sgmv_shrink_kernel<DT, RMAX>), dim3(a.max_tiles, a.ksplit), dim3(SG_NT), 0, s, a);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    {
        const long long n = (long long)a.T * (RMAX / 8);
        hipLaunchKernelGGL((sgmv_reduce_kernel<DT, RMAX>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, a);
        rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    // 512 columns per workgroup amortise the V operand; fewer when that leaves the chip idle
    int cols = 512;
    while (cols > TN && (long long)a.max_tiles * ((a.hout + cols - 1) / cols) < 1024) cols >>= 1;
    const int ncb = (a.hout + cols - 1) / cols;
    if (a.b_transposed)
        hipLaunchKernelGGL((sgmv_expand_kernel<DT, RMAX, true>), dim3(a.max_tiles, ncb), dim3(SG_NT), 0, s, a, cols);
    else
        hipLaunchKernelGGL((sgmv_expand_kernel<DT, RMAX, false>), dim3(a.max_tiles, ncb), dim3(SG_NT), 0, s, a, cols);
    return (int)hipGetLastError();
}

template <int DT>
static int launch_sg_dt(const SgmvArgs &a, int max_rank, hipStream_t s)
{
    if (max_rank <= 16) return launch_rmax<DT, 16>(a, s);
    if (max_rank <= 32) return launch_rmax<DT, 32>(a, s);
    return launch_rmax<DT, 64>(a, s);
}

int launch_sgmv(const SgmvArgs &a, int dtype, int max_rank, hipStream_t s)
{
    if (dtype == DT_F16) return launch_sg_dt<DT_F16>(a, max_rank, s);
    return launch_sg_dt<DT_BF16>(a, max_rank, s);
}

}  // namespace mlora
