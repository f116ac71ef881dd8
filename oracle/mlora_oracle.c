/*
 * mlora_oracle.c -- CPU restatement of the multi-LoRA batched-apply path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; it is never linked into, imported by, or called from the
 * shipped library or its Python host layer.  Only tests, the smoke check and
 * the benchmark's cpu_baseline leg load it.
 *
 * Every function restates, in plain scalar C, what the reference computes on
 * this path.  The reference's decode arithmetic lives in a third-party module
 * (punica==0.2.0, requirements.txt:75) that is not in the reference tree, so
 * that call is restated from its call sites and documented contract
 * (lightllm/models/lora_gpu.py:138,150,162:
 *     y[i] += x[i] @ wa_T_all[idx[i], layer].T @ wb_T_all[idx[i], layer].T * scale)
 * -- parity against punica's own outputs is UNPINNED (no vectors exist); what
 * is pinned, by the tests under tests/, is this file against closed forms,
 * brute force, library matmuls and invariants.
 *
 * Pinned functions (see tests/test_oracle_*.py):
 *   orc_f16_to_f32 / orc_f32_to_f16 / orc_bf16_* : exhaustive / randomized vs numpy & torch
 *   orc_pool_gather, orc_build_segments, orc_build_chunks, orc_build_work, orc_sgmv_plan : vs numpy closed forms / enumeration
 *   orc_pool_scatter          : numpy fancy-index assignment
 *   orc_lora_apply_paged      : brute-force fp64 loops, one-hot, scale 0, library matmul
 *   orc_gemm_lora_paged       : numpy matmul (fp64) of base product plus delta, integer-valued exact case, both rounding contracts
 *   orc_add_lora_bgmv_ref     : same expression through numpy on the reference layout
 *   orc_prefill_bmm_ref       : numpy matmul pairs (the reference's bmm.bmm)
 *   orc_cpu_lora_worker       : numpy fp32 matmul of the reference's one-line arithmetic
 *   orc_cpu_chunk_plan        : enumeration of the reference's chunk index arithmetic
 *   orc_cpu_lora_batch, orc_cpu_pool_run : the worker applied chunk by chunk / each other, bit for bit
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdlib.h>
#include <math.h>
#include <pthread.h>
#ifdef __F16C__
#include <immintrin.h>
#endif

#define ORC_OK 0
#define ORC_EINVAL (-1)
#define ORC_ERANGE (-2)

/* ------------------------------------------------------------------ */
/* 16-bit float conversions (IEEE binary16 and bfloat16), RNE.         */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t orc_f32_to_f16(float f)
{
    uint32_t u = f32_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) {                    /* inf / nan */
        if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);   /* rounds to >= 65520 -> inf */
    if (a < 0x33000001u) return sign;          /* below half of the smallest subnormal */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;  /* 24-bit significand */
    int shift;
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }          /* subnormal result */
    else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));      /* carry into the exponent is correct by construction */
}

float orc_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  /* quiet nan */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float ld16(const uint16_t *p, size_t i, int dtype)
{
    return dtype == 0 ? orc_f16_to_f32(p[i]) : orc_bf16_to_f32(p[i]);
}
static inline uint16_t st16(float v, int dtype)
{
    return dtype == 0 ? orc_f32_to_f16(v) : orc_f32_to_bf16(v);
}

/* vector helpers so that tests can pin the conversions wholesale */
void orc_f16_to_f32_n(const uint16_t *in, float *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(in[i]); }
void orc_f32_to_f16_n(const float *in, uint16_t *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(in[i]); }
void orc_bf16_to_f32_n(const uint16_t *in, float *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_bf16_to_f32(in[i]); }
void orc_f32_to_bf16_n(const float *in, uint16_t *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_bf16(in[i]); }

/* ------------------------------------------------------------------ */
/* Adapter-pool index / offset gather.                                 */
/* The reference keeps a dense pool indexed [adapter, layer, ...]       */
/* (lightllm/models/lora_gpu.py:33-40) and a per-token index vector     */
/* (lora_gpu.py:120,124).  The paged pool generalises that: rank row j  */
/* of adapter i lives at row  page_tbl[i][j / page_rows] * page_rows    */
/* + j % page_rows.  Out-of-range adapters are an error here (the       */
/* reference would read out of bounds, lora_gpu.py:120 vs manager.py:88)*/
/* and a negative adapter means "no adapter for this token".           */
/* ------------------------------------------------------------------ */

int orc_pool_gather(const int32_t *tok_adapter, int T,
                    const int32_t *page_tbl, const int32_t *rank, const float *scaling,
                    int n_adapters, int max_pages, int page_rows,
                    int32_t *out_row_off /* [T, max_pages] */, int32_t *out_rank /* [T] */,
                    float *out_scale /* [T] */)
{
    if (T < 0 || n_adapters < 0 || max_pages <= 0 || page_rows <= 0) return ORC_EINVAL;
    for (int t = 0; t < T; t++) {
        int a = tok_adapter[t];
        if (a >= n_adapters) return ORC_ERANGE;
        if (a < 0) {
            out_rank[t] = 0;
            out_scale[t] = 0.0f;
            for (int p = 0; p < max_pages; p++) out_row_off[(size_t)t * max_pages + p] = -1;
            continue;
        }
        int r = rank[a];
        int np = (r + page_rows - 1) / page_rows;
        if (np > max_pages) return ORC_ERANGE;
        out_rank[t] = r;
        out_scale[t] = scaling[a];
        for (int p = 0; p < max_pages; p++)
            out_row_off[(size_t)t * max_pages + p] = p < np ? page_tbl[(size_t)a * max_pages + p] * page_rows : -1;
    }
    return ORC_OK;
}

/* Adapter swap-in: rank row k of a contiguous block goes to slab row
 * pages[k / page_rows] * page_rows + k % page_rows (what replaces the per-layer tensor
 * copies of shared_tensor.py:117-147 / lora_gpu.py:165-188).  Plain byte copy. */
int orc_pool_scatter(const unsigned char *src, unsigned char *dst_slab, int64_t row_bytes,
                     const int32_t *pages, int n_slot_pages, int rank, int page_rows, int64_t n_pages)
{
    if (rank < 0 || page_rows <= 0 || row_bytes <= 0) return ORC_EINVAL;
    if ((rank + page_rows - 1) / page_rows > n_slot_pages) return ORC_ERANGE;
    for (int k = 0; k < rank; k++) {
        int pg = pages[k / page_rows];
        if (pg < 0 || pg >= n_pages) return ORC_ERANGE;
        int64_t row = (int64_t)pg * page_rows + k % page_rows;
        memcpy(dst_slab + row * row_bytes, src + (int64_t)k * row_bytes, (size_t)row_bytes);
    }
    return ORC_OK;
}

/* Stable grouping of tokens by adapter: perm lists token ids ordered by
 * (adapter, token id); tokens with a negative adapter come last and belong to
 * no segment.  Segments are runs of equal adapter in that order, ascending in
 * adapter id.  Returns the number of tokens that have an adapter in *n_valid. */
int orc_build_segments(const int32_t *tok_adapter, int T, int n_adapters,
                       int32_t *perm /* [T] */, int32_t *seg_start, int32_t *seg_len,
                       int32_t *seg_adapter /* each [min(T, n_adapters)] */,
                       int32_t *n_seg, int32_t *n_valid)
{
    if (T < 0 || n_adapters < 0) return ORC_EINVAL;
    int32_t *count = (int32_t *)calloc((size_t)n_adapters + 1, sizeof(int32_t));
    int32_t *start = (int32_t *)calloc((size_t)n_adapters + 1, sizeof(int32_t));
    if (!count || !start) { free(count); free(start); return ORC_EINVAL; }
    int valid = 0;
    for (int t = 0; t < T; t++) {
        int a = tok_adapter[t];
        if (a >= n_adapters) { free(count); free(start); return ORC_ERANGE; }
        if (a >= 0) { count[a]++; valid++; }
    }
    int ns = 0, pos = 0;
    for (int a = 0; a < n_adapters; a++) {
        start[a] = pos;
        if (count[a] > 0) {
            seg_start[ns] = pos; seg_len[ns] = count[a]; seg_adapter[ns] = a; ns++;
        }
        pos += count[a];
    }
    int tail = valid;
    for (int t = 0; t < T; t++) {                 /* ascending t => stable */
        int a = tok_adapter[t];
        if (a >= 0) perm[start[a]++] = t; else perm[tail++] = t;
    }
    *n_seg = ns; *n_valid = valid;
    free(count); free(start);
    return ORC_OK;
}

/* Decode work list: every segment is cut into chunks of at most `group`
 * tokens; chunk c covers sorted positions [chunk_start[c], chunk_start[c] +
 * chunk_len[c]) and uses chunk_adapter[c].  Tokens without an adapter form
 * trailing chunks with adapter -1 (they only matter when the caller asks for
 * y = delta, where their rows must be written as zero). */
int orc_build_chunks(const int32_t *seg_start, const int32_t *seg_len, const int32_t *seg_adapter,
                     int n_seg, int n_valid, int T, int group,
                     int32_t *chunk_start, int32_t *chunk_len, int32_t *chunk_adapter, int32_t *n_chunks)
{
    if (group <= 0) return ORC_EINVAL;
    int nc = 0;
    for (int s = 0; s < n_seg; s++)
        for (int o = 0; o < seg_len[s]; o += group) {
            chunk_start[nc] = seg_start[s] + o;
            chunk_len[nc] = seg_len[s] - o < group ? seg_len[s] - o : group;
            chunk_adapter[nc] = seg_adapter[s];
            nc++;
        }
    for (int o = n_valid; o < T; o += group) {
        chunk_start[nc] = o;
        chunk_len[nc] = T - o < group ? T - o : group;
        chunk_adapter[nc] = -1;
        nc++;
    }
    *n_chunks = nc;
    return ORC_OK;
}

/* Decode work records for the fused decode kernel, in launch order.  Chunk c is served by the
 * workgroup b = (c mod per_xcd) * 8 + c / per_xcd with per_xcd = ceil(n_chunks / 8): workgroups are
 * dealt to the 8 XCDs round-robin by id, so consecutive chunks land on one XCD.  Record b
 * (ORC_WORK_WORDS int32): [0] tokens in the chunk (0 = empty record), [1] adapter (-1 = none),
 * [2] rank clamped to 0..64, [3] scaling as float bits, [4..11] token ids (-1 unused), [12..15] 0,
 * [16..79] row of rank row j = page_tbl[a][j / page_rows] * page_rows + j % page_rows, or -1 when
 * j >= rank or the page id is outside [0, n_pages).  This is layout bookkeeping of this build (the
 * reference has no counterpart); it is pinned by direct enumeration in the tests. */
#define ORC_WORK_WORDS 80
int orc_build_work(const int32_t *chunk_start, const int32_t *chunk_len, const int32_t *chunk_adapter,
                   int n_chunks, const int32_t *perm, const int32_t *page_tbl, const int32_t *rank,
                   const float *scaling, int max_pages, int page_rows, int64_t n_pages,
                   int work_cap, int32_t *work /* [work_cap * ORC_WORK_WORDS] */)
{
    if (work_cap < 0 || (work_cap & 7) || n_chunks > work_cap) return ORC_EINVAL;
    int per_xcd = (n_chunks + 7) / 8;
    for (int b = 0; b < work_cap; b++) {
        int32_t *w = work + (size_t)b * ORC_WORK_WORDS;
        for (int i = 0; i < ORC_WORK_WORDS; i++) w[i] = 0;
        w[1] = -1;
    }
    /* Batches of at most 2048 tokens (work_cap <= 2048): inside the range of chunks that goes to one XCD the
     * records follow falling rank, ties in chunk order (a stable insertion sort per range). */
    int *ord = (int *)malloc((size_t)(n_chunks > 0 ? n_chunks : 1) * sizeof(int));
    int *crk = (int *)malloc((size_t)(n_chunks > 0 ? n_chunks : 1) * sizeof(int));
    if (!ord || !crk) { free(ord); free(crk); return ORC_EINVAL; }
    for (int c = 0; c < n_chunks; c++) {
        int a = chunk_adapter[c], rk = 0;
        if (a >= 0) { rk = rank[a]; if (rk < 0) rk = 0; if (rk > 64) rk = 64; }
        crk[c] = rk;
        ord[c] = c;
    }
    if (work_cap <= 2048) {
        for (int lo = 0; lo < n_chunks; lo += per_xcd) {
            int hi = lo + per_xcd < n_chunks ? lo + per_xcd : n_chunks;
            for (int i = lo + 1; i < hi; i++) {
                int c = ord[i], j = i;
                while (j > lo && crk[ord[j - 1]] < crk[c]) { ord[j] = ord[j - 1]; j--; }
                ord[j] = c;
            }
        }
    }
    for (int pos = 0; pos < n_chunks; pos++) {
        int c = ord[pos];
        int b = (pos % per_xcd) * 8 + pos / per_xcd;
        int32_t *w = work + (size_t)b * ORC_WORK_WORDS;
        int a = chunk_adapter[c];
        int rk = crk[c];
        w[0] = chunk_len[c];
        w[1] = a;
        w[2] = rk;
        if (a >= 0) memcpy(&w[3], &scaling[a], 4);
        for (int k = 0; k < 8; k++) w[4 + k] = k < chunk_len[c] ? perm[chunk_start[c] + k] : -1;
        for (int j = 0; j < 64; j++) {
            int32_t v = -1;
            if (a >= 0 && j < rk && j / page_rows < max_pages) {
                int32_t pg = page_tbl[(size_t)a * max_pages + j / page_rows];
                if (pg >= 0 && pg < n_pages) v = pg * page_rows + j % page_rows;
            }
            w[16 + j] = v;
        }
    }
    free(ord);
    free(crk);
    return ORC_OK;
}

/* Prefill work list: every segment (a request's contiguous tokens, as the
 * reference batches one adapter slot per request, lora_gpu.py:125-128) is cut
 * into tiles of `tile` tokens.  tile_seg / tile_tok0 / tile_ntok per tile. */
int orc_sgmv_plan(const int32_t *seg_start, const int32_t *seg_len, int n_seg, int tile,
                  int32_t *tile_seg, int32_t *tile_tok0, int32_t *tile_ntok, int32_t *n_tiles)
{
    if (tile <= 0) return ORC_EINVAL;
    int nt = 0;
    for (int s = 0; s < n_seg; s++)
        for (int o = 0; o < seg_len[s]; o += tile) {
            tile_seg[nt] = s;
            tile_tok0[nt] = seg_start[s] + o;
            tile_ntok[nt] = seg_len[s] - o < tile ? seg_len[s] - o : tile;
            nt++;
        }
    *n_tiles = nt;
    return ORC_OK;
}

/* The same with the cuts at multiples of `tile` tokens (and at segment ends): segment [start, start + len) gives
 * the non-empty pieces [max(start, k tile), min(start + len, (k + 1) tile)), k ascending. */
int orc_sgmv_plan_aligned(const int32_t *seg_start, const int32_t *seg_len, int n_seg, int tile,
                          int32_t *tile_seg, int32_t *tile_tok0, int32_t *tile_ntok, int32_t *n_tiles)
{
    if (tile <= 0) return ORC_EINVAL;
    int nt = 0;
    for (int s = 0; s < n_seg; s++) {
        int b = seg_start[s], end = seg_start[s] + seg_len[s];
        while (b < end) {
            int e = (b / tile + 1) * tile;
            if (e > end) e = end;
            tile_seg[nt] = s; tile_tok0[nt] = b; tile_ntok[nt] = e - b;
            nt++;
            b = e;
        }
    }
    *n_tiles = nt;
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* LoRA apply over the paged pool:                                     */
/*   y[t] = round16( y0[t] + s_a * (x[t] . A_a) . B_a ),  a = adapter   */
/* A rows are rank rows of length Hin (A^T), B rows are rank rows of    */
/* length Hout; accumulation in fp32 (acc64 = 0) or fp64 (acc64 = 1),   */
/* one rounding to the 16-bit type at the end.  The reference rounds    */
/* the delta first and adds in fp16 (lora_gpu.py:137-138 then           */
/* transformer_layer_infer.py:160-171); single rounding is the stated   */
/* contract of this build and differs by at most one ulp of y.          */
/* y0 == NULL means y = delta.                                         */
/* ------------------------------------------------------------------ */

int orc_lora_apply_paged(uint16_t *y, const uint16_t *y0, const uint16_t *x,
                         const uint16_t *a_rows, const uint16_t *b_rows,
                         const int32_t *tok_adapter,
                         const int32_t *a_page_tbl, const int32_t *b_page_tbl,
                         const int32_t *rank, const float *scaling,
                         int T, int Hin, int Hout, int n_adapters, int max_pages, int page_rows,
                         int dtype, int acc64)
{
    if (T < 0 || Hin <= 0 || Hout <= 0 || max_pages <= 0 || page_rows <= 0) return ORC_EINVAL;
    if (dtype != 0 && dtype != 1) return ORC_EINVAL;
    for (int t = 0; t < T; t++) {
        int a = tok_adapter[t];
        if (a >= n_adapters) return ORC_ERANGE;
        if (a >= 0 && (rank[a] + page_rows - 1) / page_rows > max_pages) return ORC_ERANGE;
    }
    double *vd = (double *)malloc(sizeof(double) * (size_t)max_pages * page_rows);
    float *vf = (float *)malloc(sizeof(float) * (size_t)max_pages * page_rows);
    if (!vd || !vf) { free(vd); free(vf); return ORC_EINVAL; }
    for (int t = 0; t < T; t++) {
        int a = tok_adapter[t];
        const uint16_t *xt = x + (size_t)t * Hin;
        uint16_t *yt = y + (size_t)t * Hout;
        if (a < 0) {
            for (int c = 0; c < Hout; c++) yt[c] = y0 ? y0[(size_t)t * Hout + c] : 0;
            continue;
        }
        int r = rank[a];
        float s = scaling[a];
        for (int j = 0; j < r; j++) {
            size_t row = (size_t)a_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
            const uint16_t *ar = a_rows + row * Hin;
            if (acc64) {
                double acc = 0.0;
                for (int k = 0; k < Hin; k++) acc += (double)ld16(xt, k, dtype) * (double)ld16(ar, k, dtype);
                vd[j] = acc;
            } else {
                float acc = 0.0f;
                for (int k = 0; k < Hin; k++) acc += ld16(xt, k, dtype) * ld16(ar, k, dtype);
                vf[j] = acc;
            }
        }
        for (int c = 0; c < Hout; c++) {
            if (acc64) {
                double acc = 0.0;
                for (int j = 0; j < r; j++) {
                    size_t row = (size_t)b_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
                    acc += vd[j] * (double)ld16(b_rows + row * Hout, c, dtype);
                }
                double base = y0 ? (double)ld16(y0 + (size_t)t * Hout, c, dtype) : 0.0;
                yt[c] = st16((float)(base + (double)s * acc), dtype);
            } else {
                float acc = 0.0f;
                for (int j = 0; j < r; j++) {
                    size_t row = (size_t)b_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
                    acc += vf[j] * ld16(b_rows + row * Hout, c, dtype);
                }
                float base = y0 ? ld16(y0 + (size_t)t * Hout, c, dtype) : 0.0f;
                yt[c] = st16(base + s * acc, dtype);
            }
        }
    }
    free(vd); free(vf);
    return ORC_OK;
}

/* Base projection plus LoRA delta (lightllm/models/llama/layer_infer/transformer_layer_infer.py:145-147 then
 * :160-171, with q_weight_ stored as [Hin, Hout], layer_weights/transformer_layer_weight.py:44-46):
 *     q = torch.mm(x, Wq);  q += q_lora
 * ref_rounding = 1 restates the reference's three roundings (mm result to 16 bits, delta to 16 bits, their
 * sum to 16 bits); ref_rounding = 0 is this build's contract: base product and delta summed in fp32 and
 * rounded once.  Accumulation in fp32 (acc64 = 0, ascending k) or fp64 (acc64 = 1).  Tokens with a negative
 * adapter get the base product alone. */
int orc_gemm_lora_paged(uint16_t *y, const uint16_t *x, const uint16_t *w,
                        const uint16_t *a_rows, const uint16_t *b_rows, const int32_t *tok_adapter,
                        const int32_t *a_page_tbl, const int32_t *b_page_tbl, const int32_t *rank, const float *scaling,
                        int T, int Hin, int Hout, int n_adapters, int max_pages, int page_rows,
                        int dtype, int acc64, int ref_rounding)
{
    if (T < 0 || Hin <= 0 || Hout <= 0 || max_pages <= 0 || page_rows <= 0) return ORC_EINVAL;
    if (dtype != 0 && dtype != 1) return ORC_EINVAL;
    for (int t = 0; t < T; t++) {
        int a = tok_adapter[t];
        if (a >= n_adapters) return ORC_ERANGE;
        if (a >= 0 && (rank[a] + page_rows - 1) / page_rows > max_pages) return ORC_ERANGE;
    }
    double *base = (double *)malloc(sizeof(double) * (size_t)Hout);
    float *basef = (float *)malloc(sizeof(float) * (size_t)Hout);
    double *v = (double *)malloc(sizeof(double) * (size_t)max_pages * page_rows);
    if (!base || !basef || !v) { free(base); free(basef); free(v); return ORC_EINVAL; }
    for (int t = 0; t < T; t++) {
        const uint16_t *xt = x + (size_t)t * Hin;
        for (int c = 0; c < Hout; c++) { base[c] = 0.0; basef[c] = 0.0f; }
        for (int k = 0; k < Hin; k++) {
            const float xv = ld16(xt, k, dtype);
            const uint16_t *wr = w + (size_t)k * Hout;
            if (acc64) for (int c = 0; c < Hout; c++) base[c] += (double)xv * (double)ld16(wr, c, dtype);
            else for (int c = 0; c < Hout; c++) basef[c] += xv * ld16(wr, c, dtype);
        }
        if (!acc64) for (int c = 0; c < Hout; c++) base[c] = basef[c];
        int a = tok_adapter[t];
        int r = a >= 0 ? rank[a] : 0;
        for (int j = 0; j < r; j++) {
            size_t row = (size_t)a_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
            const uint16_t *ar = a_rows + row * Hin;
            if (acc64) {
                double acc = 0.0;
                for (int k = 0; k < Hin; k++) acc += (double)ld16(xt, k, dtype) * (double)ld16(ar, k, dtype);
                v[j] = acc;
            } else {
                float acc = 0.0f;
                for (int k = 0; k < Hin; k++) acc += ld16(xt, k, dtype) * ld16(ar, k, dtype);
                v[j] = acc;
            }
        }
        for (int c = 0; c < Hout; c++) {
            double d = 0.0;
            if (acc64) {
                for (int j = 0; j < r; j++) {
                    size_t row = (size_t)b_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
                    d += v[j] * (double)ld16(b_rows + row * Hout, c, dtype);
                }
                if (a >= 0) d *= (double)scaling[a];
            } else {
                float acc = 0.0f;
                for (int j = 0; j < r; j++) {
                    size_t row = (size_t)b_page_tbl[(size_t)a * max_pages + j / page_rows] * page_rows + j % page_rows;
                    acc += (float)v[j] * ld16(b_rows + row * Hout, c, dtype);
                }
                d = a >= 0 ? (double)(scaling[a] * acc) : 0.0;
            }
            uint16_t out;
            if (ref_rounding) {
                uint16_t q = st16((float)base[c], dtype);
                if (a >= 0) {
                    uint16_t ql = st16((float)d, dtype);
                    uint16_t one = q;
                    q = st16(ld16(&one, 0, dtype) + ld16(&ql, 0, dtype), dtype);
                }
                out = q;
            } else {
                out = acc64 ? st16((float)(base[c] + d), dtype) : st16((float)base[c] + (float)d, dtype);
            }
            y[(size_t)t * Hout + c] = out;
        }
    }
    free(base); free(basef); free(v);
    return ORC_OK;
}

/* The reference's decode call on the reference's own layout
 * (lora_gpu.py:33-40,137-138): wa_T_all [N, L, r, Hin], wb_T_all [N, L, Hout, r],
 * fp16, indices int64 [T];  y[t] += scale * (x[t] . wa[idx,layer]^T) . wb[idx,layer]^T. */
int orc_add_lora_bgmv_ref(uint16_t *y, const uint16_t *x,
                          const uint16_t *wa_T_all, const uint16_t *wb_T_all,
                          const int64_t *indices, int T, int N, int L, int r,
                          int Hin, int Hout, int layer_idx, float scale, int dtype)
{
    if (layer_idx < 0 || layer_idx >= L || r <= 0) return ORC_EINVAL;
    float *v = (float *)malloc(sizeof(float) * (size_t)r);
    if (!v) return ORC_EINVAL;
    for (int t = 0; t < T; t++) {
        int64_t a = indices[t];
        if (a < 0 || a >= N) { free(v); return ORC_ERANGE; }
        const uint16_t *wa = wa_T_all + ((size_t)a * L + layer_idx) * (size_t)r * Hin;
        const uint16_t *wb = wb_T_all + ((size_t)a * L + layer_idx) * (size_t)Hout * r;
        for (int j = 0; j < r; j++) {
            float acc = 0.0f;
            for (int k = 0; k < Hin; k++) acc += ld16(x + (size_t)t * Hin, k, dtype) * ld16(wa + (size_t)j * Hin, k, dtype);
            v[j] = acc;
        }
        for (int c = 0; c < Hout; c++) {
            float acc = 0.0f;
            for (int j = 0; j < r; j++) acc += v[j] * ld16(wb + (size_t)c * r, j, dtype);
            size_t o = (size_t)t * Hout + c;
            y[o] = st16(ld16(y, o, dtype) + scale * acc, dtype);
        }
    }
    free(v);
    return ORC_OK;
}

/* The reference's prefill call (lora_gpu.py:125-128): request b uses adapter
 * slot b; x [B, Lpad, Hin]; A_T [B, L, r, Hin]; B_T [B, L, Hout, r];
 * y = bmm(bmm(x, A), B).  torch.bmm on fp16 stores its result in fp16, so the
 * reference rounds the [B, Lpad, r] intermediate; round_mid = 1 restates that,
 * round_mid = 0 keeps it in fp32 (this build's contract). */
int orc_prefill_bmm_ref(uint16_t *y, const uint16_t *x, const uint16_t *A_T, const uint16_t *B_T,
                        int Bsz, int Lpad, int L, int r, int Hin, int Hout, int layer_idx,
                        int dtype, int round_mid)
{
    if (layer_idx < 0 || layer_idx >= L || r <= 0) return ORC_EINVAL;
    float *v = (float *)malloc(sizeof(float) * (size_t)r);
    if (!v) return ORC_EINVAL;
    for (int b = 0; b < Bsz; b++) {
        const uint16_t *wa = A_T + ((size_t)b * L + layer_idx) * (size_t)r * Hin;
        const uint16_t *wb = B_T + ((size_t)b * L + layer_idx) * (size_t)Hout * r;
        for (int l = 0; l < Lpad; l++) {
            const uint16_t *xt = x + ((size_t)b * Lpad + l) * Hin;
            for (int j = 0; j < r; j++) {
                float acc = 0.0f;
                for (int k = 0; k < Hin; k++) acc += ld16(xt, k, dtype) * ld16(wa + (size_t)j * Hin, k, dtype);
                v[j] = round_mid ? ld16((uint16_t[]){st16(acc, dtype)}, 0, dtype) : acc;
            }
            for (int c = 0; c < Hout; c++) {
                float acc = 0.0f;
                for (int j = 0; j < r; j++) acc += v[j] * ld16(wb + (size_t)c * r, j, dtype);
                y[((size_t)b * Lpad + l) * Hout + c] = st16(acc, dtype);
            }
        }
    }
    free(v);
    return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* The CPU-assisted path's arithmetic (lora_cpu/lora_shm_op/app.py:     */
/* 133-141): one worker takes a chunk of at most `cap` tokens of one    */
/* request and one projection and computes                              */
/*     res = x.float() @ down @ up ;  out = res.half()                  */
/* with fp32 weights down [Hin, r], up [r, Hout] (app.py:38-45).        */
/* ------------------------------------------------------------------ */

/* fp16 <-> fp32 of whole rows.  With F16C the hardware conversions are used (IEEE, round to nearest
 * even: the same values as orc_f16_to_f32 / orc_f32_to_f16 for every finite input and infinity). */
static void orc_row_f16_to_f32(const uint16_t *src, float *dst, int n)
{
    int i = 0;
#ifdef __F16C__
    for (; i + 8 <= n; i += 8)
        _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(src + i))));
#endif
    for (; i < n; i++) dst[i] = orc_f16_to_f32(src[i]);
}

static void orc_row_f32_to_f16(const float *src, uint16_t *dst, int n)
{
    int i = 0;
#ifdef __F16C__
    for (; i + 8 <= n; i += 8)
        _mm_storeu_si128((__m128i *)(dst + i), _mm256_cvtps_ph(_mm256_loadu_ps(src + i), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
#endif
    for (; i < n; i++) dst[i] = orc_f32_to_f16(src[i]);
}

int orc_cpu_lora_worker(const uint16_t *x /* [n_tok, Hin] fp16 */, const float *down, const float *up,
                        uint16_t *out /* [n_tok, Hout] fp16 */, int n_tok, int Hin, int Hout, int r)
{
    if (n_tok < 0 || r <= 0) return ORC_EINVAL;
    float *tmp = (float *)malloc(sizeof(float) * ((size_t)r + (size_t)Hout + (size_t)Hin));
    if (!tmp) return ORC_EINVAL;
    float *row = tmp + r, *xf = row + Hout;
    for (int t = 0; t < n_tok; t++) {
        orc_row_f16_to_f32(x + (size_t)t * Hin, xf, Hin);
        for (int j = 0; j < r; j++) tmp[j] = 0.0f;
        for (int k = 0; k < Hin; k++) {
            float xv = xf[k];
            const float *d = down + (size_t)k * r;
            for (int j = 0; j < r; j++) tmp[j] += xv * d[j];
        }
        for (int c = 0; c < Hout; c++) row[c] = 0.0f;
        for (int j = 0; j < r; j++) {
            const float *u = up + (size_t)j * Hout;
            float tv = tmp[j];
            for (int c = 0; c < Hout; c++) row[c] += tv * u[c];
        }
        orc_row_f32_to_f16(row, out + (size_t)t * Hout, Hout);
    }
    free(tmp);
    return ORC_OK;
}

/* Chunk arithmetic of the CPU-assisted path.  The driver cuts each request's
 * tkn_num tokens into cpu_per_request = (tkn_num-1)/cap + 1 chunks
 * (lightllm/models/lora_cpu.py:150-151); worker `row_id` serves request
 * dim_0 = row_id / cpu_per_request, chunk dim_1 = row_id % cpu_per_request,
 * tokens [dim_1*cap, min((dim_1+1)*cap, tkn_num)) (app.py:133-136, restated
 * from the math: the reference clips tkn_num to cap before the worker sees it,
 * lora_cpu.py:175, which only agrees with this when a request fits one chunk).
 * The collector places chunk (b, dim_1) at token offset dim_1*cap of request b,
 * last chunk holding tkn_num - (cpr-1)*cap tokens (lora_cpu.py:210-232). */
int orc_cpu_chunk_plan(int batch, int tkn_num, int cap,
                       int32_t *req /* [batch*cpr] */, int32_t *tok0, int32_t *ntok, int32_t *n_chunks)
{
    if (batch < 0 || tkn_num <= 0 || cap <= 0) return ORC_EINVAL;
    int cpr = (tkn_num - 1) / cap + 1;
    int n = 0;
    for (int row_id = 0; row_id < batch * cpr; row_id++) {
        int d0 = row_id / cpr, d1 = row_id % cpr;
        int end = (d1 + 1) * cap < tkn_num ? (d1 + 1) * cap : tkn_num;
        req[n] = d0; tok0[n] = d1 * cap; ntok[n] = end - d1 * cap; n++;
    }
    *n_chunks = n;
    return ORC_OK;
}

/* Whole CPU-assisted LoRA delta for one projection over a batch of equal-length
 * requests, sharded as the reference shards it: one task per (request, chunk),
 * tasks spread over n_threads pinned-worker stand-ins.  Request b uses adapter
 * req_adapter[b] of the fp32 weight sets down[N][Hin][r], up[N][r][Hout].
 * Used for the benchmark's cpu_baseline leg and checked against
 * orc_cpu_lora_worker applied chunk by chunk. */
typedef struct {
    const uint16_t *x; const float *down; const float *up; uint16_t *out;
    const int32_t *req_adapter; const int32_t *req; const int32_t *tok0; const int32_t *ntok;
    int n_chunks, tkn_num, Hin, Hout, r, tid, n_threads;
} orc_cpu_job;

static void *orc_cpu_thread(void *arg)
{
    orc_cpu_job *j = (orc_cpu_job *)arg;
    for (int c = j->tid; c < j->n_chunks; c += j->n_threads) {
        int b = j->req[c];
        size_t tok = (size_t)b * j->tkn_num + j->tok0[c];
        int a = j->req_adapter[b];
        orc_cpu_lora_worker(j->x + tok * j->Hin,
                            j->down + (size_t)a * j->Hin * j->r, j->up + (size_t)a * j->r * j->Hout,
                            j->out + tok * j->Hout, j->ntok[c], j->Hin, j->Hout, j->r);
    }
    return NULL;
}

int orc_cpu_lora_batch(const uint16_t *x, const float *down, const float *up, uint16_t *out,
                       const int32_t *req_adapter, int batch, int tkn_num, int cap,
                       int Hin, int Hout, int r, int n_threads)
{
    if (n_threads <= 0 || n_threads > 256) return ORC_EINVAL;
    int cpr = (tkn_num - 1) / cap + 1;
    int32_t *req = (int32_t *)malloc(sizeof(int32_t) * 3 * (size_t)batch * cpr);
    if (!req) return ORC_EINVAL;
    int32_t *tok0 = req + (size_t)batch * cpr, *ntok = tok0 + (size_t)batch * cpr;
    int32_t nc = 0;
    int rc = orc_cpu_chunk_plan(batch, tkn_num, cap, req, tok0, ntok, &nc);
    if (rc) { free(req); return rc; }
    orc_cpu_job jobs[256];
    pthread_t th[256];
    for (int i = 0; i < n_threads; i++) {
        jobs[i] = (orc_cpu_job){x, down, up, out, req_adapter, req, tok0, ntok, nc, tkn_num, Hin, Hout, r, i, n_threads};
        if (i > 0) pthread_create(&th[i], NULL, orc_cpu_thread, &jobs[i]);
    }
    orc_cpu_thread(&jobs[0]);
    for (int i = 1; i < n_threads; i++) pthread_join(th[i], NULL);
    free(req);
    return ORC_OK;
}

/* The same batch on a persistent pool of worker threads (created once, woken per batch through a
 * mutex and condition variables), which is how the reference runs it: its workers are long-lived
 * processes pinned to cores (lora_cpu/lora_shm_op/app.py:102-167, runServerCPULoRA.py:83) and its
 * csrc thread pool is a mutex + condition-variable task queue (csrc/tpool.hpp:38-100).  Thread
 * creation is therefore not part of a timed batch.  Results are identical to orc_cpu_lora_batch. */
typedef struct orc_cpu_pool {
    pthread_mutex_t mu;
    pthread_cond_t wake, done;
    pthread_t th[256];
    int n_threads, generation, pending, stop;
    orc_cpu_job job;            /* tid / n_threads are filled per worker */
    int ids[256];
} orc_cpu_pool;

typedef struct { orc_cpu_pool *pool; int tid; } orc_pool_arg;
static orc_pool_arg orc_pool_args_storage[4][256];
static int orc_pool_slots_used = 0;

static void *orc_pool_worker(void *arg)
{
    orc_pool_arg *pa = (orc_pool_arg *)arg;
    orc_cpu_pool *p = pa->pool;
    int seen = 0;
    for (;;) {
        pthread_mutex_lock(&p->mu);
        while (!p->stop && p->generation == seen) pthread_cond_wait(&p->wake, &p->mu);
        if (p->stop) { pthread_mutex_unlock(&p->mu); return NULL; }
        seen = p->generation;
        orc_cpu_job j = p->job;
        pthread_mutex_unlock(&p->mu);
        j.tid = pa->tid; j.n_threads = p->n_threads;
        orc_cpu_thread(&j);
        pthread_mutex_lock(&p->mu);
        if (--p->pending == 0) pthread_cond_signal(&p->done);
        pthread_mutex_unlock(&p->mu);
    }
}

void *orc_cpu_pool_create(int n_threads)
{
    if (n_threads <= 0 || n_threads > 256 || orc_pool_slots_used >= 4) return NULL;
    orc_cpu_pool *p = (orc_cpu_pool *)calloc(1, sizeof(orc_cpu_pool));
    if (!p) return NULL;
    pthread_mutex_init(&p->mu, NULL);
    pthread_cond_init(&p->wake, NULL);
    pthread_cond_init(&p->done, NULL);
    p->n_threads = n_threads;
    orc_pool_arg *args = orc_pool_args_storage[orc_pool_slots_used++];
    for (int i = 0; i < n_threads; i++) {
        args[i].pool = p; args[i].tid = i;
        pthread_create(&p->th[i], NULL, orc_pool_worker, &args[i]);
    }
    return p;
}

int orc_cpu_pool_run(void *pool, const uint16_t *x, const float *down, const float *up, uint16_t *out,
                     const int32_t *req_adapter, int batch, int tkn_num, int cap, int Hin, int Hout, int r)
{
    orc_cpu_pool *p = (orc_cpu_pool *)pool;
    if (!p) return ORC_EINVAL;
    int cpr = (tkn_num - 1) / cap + 1;
    int32_t *req = (int32_t *)malloc(sizeof(int32_t) * 3 * (size_t)batch * cpr);
    if (!req) return ORC_EINVAL;
    int32_t *tok0 = req + (size_t)batch * cpr, *ntok = tok0 + (size_t)batch * cpr;
    int32_t nc = 0;
    int rc = orc_cpu_chunk_plan(batch, tkn_num, cap, req, tok0, ntok, &nc);
    if (rc) { free(req); return rc; }
    pthread_mutex_lock(&p->mu);
    p->job = (orc_cpu_job){x, down, up, out, req_adapter, req, tok0, ntok, nc, tkn_num, Hin, Hout, r, 0, p->n_threads};
    p->pending = p->n_threads;
    p->generation++;
    pthread_cond_broadcast(&p->wake);
    while (p->pending > 0) pthread_cond_wait(&p->done, &p->mu);
    pthread_mutex_unlock(&p->mu);
    free(req);
    return ORC_OK;
}

void orc_cpu_pool_destroy(void *pool)
{
    orc_cpu_pool *p = (orc_cpu_pool *)pool;
    if (!p) return;
    pthread_mutex_lock(&p->mu);
    p->stop = 1;
    pthread_cond_broadcast(&p->wake);
    pthread_mutex_unlock(&p->mu);
    for (int i = 0; i < p->n_threads; i++) pthread_join(p->th[i], NULL);
    pthread_mutex_destroy(&p->mu);
    pthread_cond_destroy(&p->wake);
    pthread_cond_destroy(&p->done);
    free(p);
}
