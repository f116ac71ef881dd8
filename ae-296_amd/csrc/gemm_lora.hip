// Base projection with the LoRA expand folded in, for gfx950 (prefill: packed tokens, one adapter per segment):
//     y[t, :] = round16( x[t, :] . W  +  s_a * (x[t, :] . A_a) . B_a )
// W is [hin, hout] row-major (the layout lightllm keeps its projection weights in:
// lightllm/models/llama/layer_weights/transformer_layer_weight.py:44-46), x is [T, hin].
// Replaces, for one layer, torch.mm(x, W) followed by `q += q_lora`
// (lightllm/models/llama/layer_infer/transformer_layer_infer.py:145-147,160-171): y is written once and
// never read, x is read once per column tile.
//
// The rank-r intermediate s_a * (x . A_a) comes from the SGMV shrink launch (sgmv_prefill.hip) and the
// scaled reduce below, as a hi + lo pair of 16-bit values per element; the kernel here treats it as
// extra K columns of the GEMM: after the K loop over W, every 32-row block of the output tile runs
// rank / 16 more MFMA steps with (intermediate, B rows of its adapter) as operands.
//
// One workgroup (256 threads, 2 x 2 wavefronts of 128 x 128 outputs each) computes a 256 x 256 tile of y
// on v_mfma_f32_32x32x16_{f16,bf16}.  K advances 32 columns per step through a ring of four LDS stages
// that global memory fills directly (buffer_load ... lds): while the MFMAs of step k run from one stage, the
// loads of steps k+1 .. k+3 are in flight or landed.  x is K-contiguous, so its operand is a plain 16-byte
// LDS read; W is N-contiguous and is read back with the transposing LDS read.
#include "mlora_args.hpp"
#include "mlora_dev.hpp"
#include <type_traits>

namespace mlora {

constexpr int GM = 256;                 // rows (tokens) per tile
constexpr int GN = 256;                 // output columns per tile
constexpr int GK = 32;                  // K columns per stage
constexpr int NST = 4;                  // stages in flight (a ring)
constexpr int G_NT = 256;
constexpr int A_BYTES = GM * GK * 2;    // x tile of a stage, rows unpadded and chunk-swizzled
constexpr int B_BYTES = GK * GN * 2;    // W tile of a stage, likewise
constexpr int STAGE = A_BYTES + B_BYTES;
constexpr int OPITCH = 128 * 2 + 16;    // bytes per row of a wavefront's 32 x 128 output staging tile
constexpr int GROUP_M = 4;              // row tiles that share W column tiles back to back on one XCD
typedef short gl_short4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) gl_short4 gl_lds_short4;

static_assert(NST * STAGE <= 160 * 1024 - 4096, "the stages and the small tables must fit the LDS of a compute unit");
static_assert(32 * OPITCH <= STAGE && MAX_RANK * GN * 2 <= STAGE, "a wavefront's output staging and the parked B rows each reuse one stage");

template <int DT>
__device__ __forceinline__ float16_t mfma32(const uint4 &a, const uint4 &b, float16_t c)
{
    if constexpr (DT == DT_F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf168_t, a), __builtin_bit_cast(bf168_t, b), c, 0, 0, 0);
}

// ------------------------------------------------------------------ scaled reduce
// vhi + vlo [t][0..RMAX) = s_a * sum over the K splits of the shrink partials, for the tokens of one plan
// tile (the scaling is folded in here because the GEMM accumulators also hold the base product).
template <int DT, int RMAX>
__global__ __launch_bounds__(256) void gemm_lora_reduce_kernel(const GemmLoraArgs p)
{
    constexpr int CPT = RMAX / 8;
    const int tile = blockIdx.x;
    if (tile >= p.n_tiles[0]) return;
    const GemmProj &pj = p.pr[blockIdx.y];
    const int32_t *__restrict__ rec = p.tile_rec + (size_t)tile * TILE_WORDS;
    const int ntok = rec[0], adapter = rec[1], tok0 = rec[4];
    if (adapter < 0 || ntok <= 0 || tok0 < 0 || tok0 + ntok > p.T) return;
    const float scale = __builtin_bit_cast(float, rec[3]);
    for (int idx = threadIdx.x; idx < ntok * CPT; idx += 256) {
        const int t = tok0 + idx / CPT, c0 = (idx % CPT) * 8;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.f;
        for (int sp = 0; sp < pj.ksplit; sp++) {
            const float4_t *vp = reinterpret_cast<const float4_t *>(pj.v + ((size_t)sp * p.T + t) * MAX_RANK + c0);
            const float4_t a = vp[0], b = vp[1];
            v[0] += a[0]; v[1] += a[1]; v[2] += a[2]; v[3] += a[3];
            v[4] += b[0]; v[5] += b[1]; v[6] += b[2]; v[7] += b[3];
        }
        uint32_t h[8], l[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float sv = scale * v[e];
            h[e] = cvt16<DT>(sv);
            l[e] = cvt16<DT>(sv - lo_f32<DT>(h[e]));
        }
        stg16(pj.vhi + (size_t)t * MAX_RANK + c0,
              make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)));
        stg16(pj.vlo + (size_t)t * MAX_RANK + c0,
              make_uint4(l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16)));
    }
}

// ------------------------------------------------------------------ GEMM + expand
template <int DT, int RMAX>
__global__ __launch_bounds__(G_NT, 1) void gemm_lora_kernel(const GemmLoraArgs p)
{
    // one array per stage: the compiler then knows that loads into one stage cannot alias the operand reads of another
    __shared__ __attribute__((aligned(16))) unsigned char smem[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char smem1[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char smem2[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char smem3[STAGE];
    __shared__ unsigned long long s_mask[2 * (G_NT / 64)];
    __shared__ int s_list[G_NT + 1];               // first plan tile of every run (of the 256 tiles looked at); [G_NT] = how many runs
    __shared__ int s_last[G_NT];                   // last plan tile of every run
    __shared__ int s_rows[4][MAX_RANK];            // row of every rank row of the (up to four) runs being applied
    __shared__ int s_span[4][2];                   // their first and one-past-last row, relative to this row block

    // ---- which projection, which tile.  Workgroups go to the 8 XCDs round-robin by id; every XCD works
    // through one contiguous range of the tile order below, in which GROUP_M row tiles sweep the column
    // tiles together, so that the tiles in flight on one XCD (one L2) share their x and W panels.
    int proj = 0;
    while (proj + 1 < p.n_proj && blockIdx.x >= p.pr[proj].end) proj++;
    const GemmProj &pj = p.pr[proj];
    const int w = (int)(blockIdx.x - (proj ? p.pr[proj - 1].end : 0u));
    const int ntn = pj.ntn, ntm = p.ntm;
    const int n_tiles_out = ntm * ntn;
    const int per_xcd = (n_tiles_out + 7) >> 3;
    const int L = (w & 7) * per_xcd + (w >> 3);
    if ((w >> 3) >= per_xcd || L >= n_tiles_out) return;
    const int grp = L / (GROUP_M * ntn), within = L - grp * (GROUP_M * ntn);
    const int rows_in_grp = ntm - grp * GROUP_M < GROUP_M ? ntm - grp * GROUP_M : GROUP_M;
    const int mt = grp * GROUP_M + within % rows_in_grp, nt = within / rows_in_grp;
    const int m0 = mt * GM, n0 = nt * GN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // uniform, and the compiler may keep it in an SGPR
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lh = lane >> 5;
    const int T = p.T, hin = pj.hin, hout = pj.hout;

    // Which rows of this block get which adapter.  A plan tile is at most 64 consecutive tokens of one segment;
    // consecutive tiles of one segment that overlap the block form a "run" (one adapter, one contiguous row
    // range), which is what the expand works on.  Asked now, for the first 256 tiles of the plan, so that the
    // answer is there when the K loop ends.  tile_hits: does tile ti overlap the block (and have an adapter);
    // its segment goes to `seg`.
    auto tile_hits = [&](int ti, int n_plan, int &seg) {
        seg = -1;
        if (ti < 0 || ti >= n_plan) return false;
        const int32_t *rec = p.tile_rec + (size_t)ti * TILE_WORDS;
        const int4 h = *reinterpret_cast<const int4 *>(rec);             // tokens, adapter, rank, scaling
        const int tok0 = rec[4];
        seg = rec[5];
        return h.y >= 0 && h.z > 0 && h.x > 0 && tok0 >= 0 && tok0 + h.x <= T && tok0 < m0 + GM && tok0 + h.x > m0;
    };
    const int n_plan = p.lora ? p.n_tiles[0] : 0;
    // s_list / s_last = first and last tile of every run among plan tiles b0 .. b0 + 255, in order (a run that
    // crosses the window's end is cut there); s_list[G_NT] = how many (two barriers inside)
    auto list_tiles = [&](int b0) {
        const int ti = b0 + tid;
        int seg, segp, segn;
        const bool hit = tile_hits(ti, n_plan, seg);
        const bool hitp = tid > 0 && tile_hits(ti - 1, n_plan, segp);
        const bool hitn = tid < G_NT - 1 && tile_hits(ti + 1, n_plan, segn);
        const bool head = hit && !(hitp && segp == seg), tail = hit && !(hitn && segn == seg);
        const unsigned long long balh = __ballot(head), balt = __ballot(tail);
        if (lane == 0) { s_mask[wave] = balh; s_mask[G_NT / 64 + wave] = balt; }
        __syncthreads();
        int beforeh = 0, beforet = 0;
        for (int w4 = 0; w4 < wave; w4++) {
            beforeh += __builtin_popcountll(s_mask[w4]);
            beforet += __builtin_popcountll(s_mask[G_NT / 64 + w4]);
        }
        const unsigned long long below = (1ull << lane) - 1;
        if (head) s_list[beforeh + __builtin_popcountll(balh & below)] = ti;
        if (tail) s_last[beforet + __builtin_popcountll(balt & below)] = ti;
        if (tid == G_NT - 1) s_list[G_NT] = beforeh + __builtin_popcountll(balh);
        __syncthreads();
    };
    // thread (q, j) = (tid / 64, tid % 64) copies rank row j's row index of run base + q into LDS, and its row span
    auto fill_rows = [&](int base, int count) {
        const int q = tid >> 6, j = tid & 63;
        if (base + q < count) {
            const int32_t *rec = p.tile_rec + (size_t)s_list[base + q] * TILE_WORDS;
            s_rows[q][j] = rec[TILE_ROWS_AT + j];
            if (j == 0) s_span[q][0] = rec[4] - m0;
            if (j == 1) {
                const int32_t *recl = p.tile_rec + (size_t)s_last[base + q] * TILE_WORDS;
                s_span[q][1] = recl[4] + recl[0] - m0;
            }
        }
    };
    if (p.lora) {
        // the first four runs: their records are fetched now, behind the K loop
        list_tiles(0);
        fill_rows(0, s_list[G_NT]);                // visible after the barrier that opens the K loop
    }
    const uint16_t *__restrict__ x = static_cast<const uint16_t *>(pj.x);
    const uint16_t *__restrict__ wgt = static_cast<const uint16_t *>(pj.w);

    // ---- global -> LDS, without passing through registers (buffer_load ... lds): each such load moves
    // 64 lanes x 16 bytes into 1 KiB of consecutive LDS, lane i to slot i.  The tiles therefore have no row
    // padding; bank conflicts are avoided by storing 16-byte chunk c of a row at position c ^ key(row), which
    // costs nothing on the way in (lane i simply fetches the chunk that belongs in slot i).
    //   x tile [256 rows][4 chunks]:  key = (row / 4) % 4   (16 operand rows of one chunk column -> 16 bank groups)
    //   W tile [32 k rows][32 chunks]: key = (k % 4) * 4     (the 4 rows of a transposing read -> 4 bank groups)
    // One load of wavefront w covers 16 rows of x (rows 16 (4 q + w) ..) or 2 rows of W (rows 2 (4 q + w) ..).
    // Rows beyond T and columns beyond hout are clamped to valid addresses; what they produce is never stored.
    const int rows_here = T - m0 < GM ? T - m0 : GM;
    unsigned aoff[4], boff[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int row = 16 * (4 * q + wave) + (lane >> 2);
        const int c = (lane & 3) ^ ((row >> 2) & 3);
        const int r = row < rows_here ? row : rows_here - 1;
        aoff[q] = ((unsigned)r * (unsigned)hin + (unsigned)c * 8u) * 2u;
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int k = 2 * (4 * q + wave) + (lane >> 5);
        const int c = (lane & 31) ^ ((k & 3) << 2);
        int col = n0 + c * 8;
        col = col < hout ? col : hout - 8;
        boff[q] = ((unsigned)k * (unsigned)hout + (unsigned)col) * 2u;
    }
    // A uniform descriptor per operand, a fixed 32-bit offset per load in a VGPR and the K advance as the scalar
    // offset: the loop spends no vector instructions on addresses.  The x descriptor starts at this tile's first
    // row; the launcher guarantees hin * hout * 2 < 4 GiB.
    const size_t x_bytes = (size_t)rows_here * hin * 2;
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(x + (size_t)m0 * hin), (short)0, (int)(x_bytes < 0xffffffffu ? x_bytes : 0xffffffffu), 0x00020000);
    const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(wgt), (short)0, (int)((size_t)hin * hout * 2), 0x00020000);
    // The loads are written as inline assembly: the compiler's own bookkeeping of loads that land in LDS waits
    // for all of them before any LDS read that follows, which would serialise the ring; here the waits are
    // explicit (GL_WAIT_LOADS below).  M0 carries the LDS address of the wavefront's 1 KiB chunk.  The compiler
    // keeps M0 as a reserved register: it rejects "m0" in a clobber list ("clobber list contains reserved
    // registers") and writes M0 itself right before each of its own uses; nothing in this kernel makes it
    // emit one (no LDS-bound load builtin, no relative register move, no message with an M0 payload), and the
    // build-time resource check fails if the kernel's code ever reads M0 outside these statements.  The
    // "memory" clobber keeps LDS and global accesses from being moved across a load.
    typedef int gl_i32x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) unsigned char lds_byte;
    auto rsrc_words = [](const void *base, size_t bytes) {
        const unsigned long long a = (unsigned long long)base;
        const gl_i32x4 r = {(int)(unsigned)a, (int)((a >> 32) & 0xffffu), (int)(bytes < 0xffffffffu ? bytes : 0xffffffffu), 0x00020000};
        return r;
    };
    const gl_i32x4 xrw = rsrc_words(x + (size_t)m0 * hin, x_bytes);
    const gl_i32x4 wrw = rsrc_words(wgt, (size_t)hin * hout * 2);
    auto dma1 = [](const gl_i32x4 &rs, unsigned lds_addr, unsigned voff, unsigned soff) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :: "s"(lds_addr), "v"(voff), "s"(rs), "s"(soff) : "memory");
    };
    // the 8 loads of one K step: 4 of x, 4 of W
    auto dma = [&](unsigned char *stage, int ks) {
        const unsigned soff_a = (unsigned)ks * (GK * 2), soff_b = (unsigned)ks * GK * (unsigned)hout * 2u;
        const unsigned base = (unsigned)(__UINTPTR_TYPE__)(lds_byte *)stage + (unsigned)wave * 1024u;
#pragma unroll
        for (int q = 0; q < 4; q++) dma1(xrw, base + q * 4096, aoff[q], soff_a);
#pragma unroll
        for (int q = 0; q < 4; q++) dma1(wrw, base + A_BYTES + q * 4096, boff[q], soff_b);
    };

    float16_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // Operand addresses inside a stage.  x: lane (row wm * 128 + 32 i + lane % 32, chunk 2 kk + lane / 32); the key
    // of the row does not depend on i.  W: lane group g = lane / 16, m = lane % 16 reads rows 16 kk + 8 (g / 2) +
    // m / 4 (+ 4), bytes of columns wn * 128 + 32 j + 16 (g % 2) + 4 (m % 4) ..; the key (m / 4) * 4 flips bits of j.
    unsigned a_at[2], b_at[4];
    {
        const int row = wm * 128 + l32, key = (l32 >> 2) & 3;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) a_at[kk] = (unsigned)(row * (GK * 2) + (((2 * kk + lh) ^ key) << 4));
        const int g = lane >> 4, m = lane & 15;
        const int krow = 8 * (g >> 1) + (m >> 2);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int c = wn * 16 + ((j ^ (m >> 2)) << 2) + (g & 1) * 2 + ((m & 3) >> 1);
            b_at[j] = (unsigned)(krow * (GN * 2) + c * 16 + (m & 1) * 8);
        }
    }
    // W operands of one K = 16 slice out of a [k rows][512 bytes] swizzled tile at `tile`.  The W-side operand of
    // a 32x32x16 MFMA: lane (n = lane % 32, k group = lane / 32) needs rows 8 * (lane / 32) + 0..7 of column n.
    // Each transposing read (ds_read_b64_tr_b16) serves a 16-lane group: lane i of the group addresses row
    // i / 4, columns 4 * (i % 4) .. + 3, and receives the four rows of column i; two reads give the eight rows.
    auto w_frags = [&](const unsigned char *tile, int kk, uint4 (&bf)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const unsigned char *src = tile + b_at[j] + kk * 16 * (GN * 2);
            const gl_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gl_lds_short4 *)src);
            const gl_short4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gl_lds_short4 *)(src + 4 * (GN * 2)));
            bf[j] = make_uint4(__builtin_bit_cast(uint2, lo).x, __builtin_bit_cast(uint2, lo).y,
                               __builtin_bit_cast(uint2, hi).x, __builtin_bit_cast(uint2, hi).y);
        }
    };
    // Operands of one K = 16 slice (4 x fragments, 4 W fragments), read one slice ahead of the MFMAs that use them.
    uint4 fa[2][4], fb[2][4];
    auto frags = [&](const unsigned char *stage, auto kk_c, uint4 (&af)[4], uint4 (&bf)[4]) {
        constexpr int kk = decltype(kk_c)::value;
#pragma unroll
        for (int i = 0; i < 4; i++) af[i] = *reinterpret_cast<const uint4 *>(stage + a_at[kk] + i * 32 * (GK * 2));
        w_frags(stage + A_BYTES, kk, bf);
    };
    auto mfma16x = [&](const uint4 (&af)[4], const uint4 (&bf)[4]) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = mfma32<DT>(af[i], bf[j], acc[i][j]);
    };
    using K0 = std::integral_constant<int, 0>;
    using K1 = std::integral_constant<int, 1>;
#define GL_FENCE() __builtin_amdgcn_sched_barrier(0)
    // Scheduling hints: one MFMA, then at most one operand read and at most one global load, so that the memory
    // instructions issue in the shadow of the MFMAs instead of in a burst between them (an MFMA occupies its pipe
    // for 32 cycles, issuing it takes 4).
#define GL_MIX(n_ds_read, n_load)                                                  \
    _Pragma("unroll") for (int n_ = 0; n_ < 16; n_++) {                              \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          \
        if (n_ < (n_ds_read)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    \
        if (n_ < (n_load)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);       \
    }
    // s_waitcnt with only the vector-memory counter set: at most n loads of this wavefront still in flight
    // (loads complete in order).
#define GL_WAIT_LOADS(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))
    // One K step of 32 columns out of stage `ks % 4`, two slices of 16.  Operand reads run one slice ahead of
    // the MFMAs.  The barrier sits between the slices: by then every wavefront has read all it needs from this
    // stage and its loads of step ks + 1 (requested three steps earlier) have landed, so the second slice's
    // operand prefetch reads the next stage, and this stage is free to receive step ks + 4 at once.
    // `steady`: steps ks + 1 .. ks + 4 all exist; otherwise the ends of the pipeline are checked.
    const gl_i32x4 brw = rsrc_words(pj.b_rows, (size_t)p.n_rows_b * hout * 2);   // the launcher guarantees < 4 GiB
    // one load = rank rows 2 jj and 2 jj + 1 (lanes 0..31 and 32..63) of tile q, jj = wave + 4 u, row indices from s_rows
    auto b_row_of = [&](int q, int u) { return s_rows[q][2 * (wave + 4 * u) + (lane >> 5)]; };
    auto b_rows_load = [&](int row, int u, unsigned lds_stage_wave) {
        const int j = 2 * (wave + 4 * u) + (lane >> 5);
        const int col = n0 + (((lane & 31) ^ ((j & 3) << 2)) << 3);
        // rows that do not exist and columns beyond hout read as zero: an offset outside the descriptor
        const unsigned voff = (row >= 0 && row < p.n_rows_b && col < hout)
                                  ? ((unsigned)row * (unsigned)hout + (unsigned)col) * 2u : 0xfffffff0u;
        dma1(brw, lds_stage_wave + u * 4096, voff, 0u);
    };
    auto k_step = [&](auto cur_c, auto steady_c, int ks, int ns) {
        constexpr int cur_i = decltype(cur_c)::value;
        constexpr bool steady = decltype(steady_c)::value;
        unsigned char *cur = cur_i == 0 ? smem : cur_i == 1 ? smem1 : cur_i == 2 ? smem2 : smem3;
        unsigned char *nxt = cur_i == 0 ? smem1 : cur_i == 1 ? smem2 : cur_i == 2 ? smem3 : smem;
        frags(cur, K1{}, fa[1], fb[1]);
        mfma16x(fa[0], fb[0]);
        GL_MIX(12, 0)
        GL_FENCE();
        const bool more_loads = steady || ks + 4 < ns, more_steps = steady || ks + 1 < ns;
        GL_WAIT_LOADS(steady ? 16 : 0);            // steady: the loads of steps ks + 2 and ks + 3 may still be in flight
        __syncthreads();
        // Second slice, scheduled by hand (the loads are assembly, which the scheduler will not interleave):
        // after MFMA n comes operand read n of the next step's first slice (4 of x, then 8 halves of W) and,
        // for n < 8, load n of step ks + 4 into the stage that has just been released.
        const unsigned soff_a = (unsigned)(ks + 4) * (GK * 2), soff_b = (unsigned)(ks + 4) * GK * (unsigned)hout * 2u;
        const unsigned lbase = (unsigned)(__UINTPTR_TYPE__)(lds_byte *)cur + (unsigned)wave * 1024u;
#pragma unroll
        for (int n = 0; n < 16; n++) {
            acc[n >> 2][n & 3] = mfma32<DT>(fa[1][n >> 2], fb[1][n & 3], acc[n >> 2][n & 3]);
            if (more_steps) {
                if (n < 4) {
                    fa[0][n] = *reinterpret_cast<const uint4 *>(nxt + a_at[0] + n * 32 * (GK * 2));
                } else if (n < 12) {
                    const int j = (n - 4) >> 1;
                    const unsigned char *src = nxt + A_BYTES + b_at[j] + ((n & 1) ? 4 * (GN * 2) : 0);
                    const uint2 h = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((gl_lds_short4 *)src));
                    if (n & 1) { fb[0][j].z = h.x; fb[0][j].w = h.y; } else { fb[0][j].x = h.x; fb[0][j].y = h.y; }
                }
            }
            if (more_loads && n < 8) {
                if (n < 4) dma1(xrw, lbase + n * 4096, aoff[n], soff_a);
                else dma1(wrw, lbase + A_BYTES + (n - 4) * 4096, boff[n - 4], soff_b);
            }
            GL_FENCE();
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    using Yes = std::true_type;
    using No = std::false_type;

    // Full K steps run through the pipeline; a partial last step follows on its own.
    const int ns = hin / GK;
    if (ns > 0) {
        dma(smem, 0);
        if (ns > 1) dma(smem1, 1);
        if (ns > 2) dma(smem2, 2);
        if (ns > 3) dma(smem3, 3);
        GL_WAIT_LOADS(0);
        __syncthreads();
        frags(smem, K0{}, fa[0], fb[0]);
        int ks = 0;
#pragma unroll 1
        for (; ks + 8 <= ns; ks += 4) {                                  // all four steps have steps ks + 4 .. behind them
            k_step(S0{}, Yes{}, ks, ns);
            k_step(S1{}, Yes{}, ks + 1, ns);
            k_step(S2{}, Yes{}, ks + 2, ns);
            k_step(S3{}, Yes{}, ks + 3, ns);
        }
#pragma unroll 1
        for (; ks < ns; ks += 4) {                                       // the last (at most seven) steps
            k_step(S0{}, No{}, ks, ns);
            if (ks + 1 < ns) k_step(S1{}, No{}, ks + 1, ns);
            if (ks + 2 < ns) k_step(S2{}, No{}, ks + 2, ns);
            if (ks + 3 < ns) k_step(S3{}, No{}, ks + 3, ns);
        }
    }
    if (ns * GK < hin) {
        // Partial last K step: through registers, with chunks of x and rows of W beyond hin replaced by zeros,
        // parked in the same swizzled layout, in the stage after the one the last full step read (some wavefronts
        // may still be reading that one; the one after it was released four steps ago).
        unsigned char *st = (ns & 3) == 0 ? smem : (ns & 3) == 1 ? smem1 : (ns & 3) == 2 ? smem2 : smem3;
        const int ncc = hin >> 3;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int row = 16 * (4 * q + wave) + (lane >> 2);
            const int c = (lane & 3) ^ ((row >> 2) & 3);
            const bool ok = ns * 4 + c < ncc;
            const unsigned back = ok ? 0u : (unsigned)(ns * 4 + c - (ncc - 1)) * 16u;
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(xrs, (int)(aoff[q] - back), ns * (GK * 2), 0);
            *reinterpret_cast<uint4 *>(st + (4 * q + wave) * 1024 + lane * 16) = ok ? make_uint4(v.x, v.y, v.z, v.w) : zero16();
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int k = ns * GK + 2 * (4 * q + wave) + (lane >> 5);
            const bool ok = k < hin;
            const unsigned back = ok ? 0u : (unsigned)(k - (hin - 1)) * (unsigned)hout * 2u;
            const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(wrs, (int)(boff[q] - back), (int)((unsigned)ns * GK * (unsigned)hout * 2u), 0);
            *reinterpret_cast<uint4 *>(st + A_BYTES + (4 * q + wave) * 1024 + lane * 16) = ok ? make_uint4(v.x, v.y, v.z, v.w) : zero16();
        }
        __syncthreads();
        const int rem = hin - ns * GK;
        frags(st, K0{}, fa[0], fb[0]); mfma16x(fa[0], fb[0]);
        if (rem > 16) { frags(st, K1{}, fa[0], fb[0]); mfma16x(fa[0], fb[0]); }
    }
    __syncthreads();                               // every wavefront is done with the stages
#undef GL_FENCE
#undef GL_MIX

    // ---- LoRA expand as extra K columns.  The plan tiles that overlap this row block (listed in LDS, 256 plan
    // tiles at a time) are handled four at a time: the B rows of each tile's adapter for this column tile go
    // straight into one of the four (now free) stages, in the W tile's layout; then every 32-row block runs, for each tile that overlaps it, RMAX / 16 slices
    // of two MFMAs per 32 columns with (hi, lo) of the intermediate of the tile's rows as the x operand (zero
    // for the other rows).  The intermediate depends on the row only, so a block's operands are read once,
    // one block ahead, whatever tiles cover it.
    if (p.lora) {
        constexpr int NSL = RMAX / 16;             // rank rows an adapter does not have read as zeros on both sides,
                                                   // so every tile runs the same RMAX / 16 slices
        // (hi, lo) of rank columns 16 s + 8 (lane / 32) .. + 7 of this lane's row in 32-row block i
        auto load_v = [&](int i, uint4 (&vh)[NSL], uint4 (&vl)[NSL]) {
            int row = m0 + wm * 128 + i * 32 + l32;
            row = row < T ? row : T - 1;
            const size_t at = (size_t)row * MAX_RANK + 8 * lh;
#pragma unroll
            for (int sl = 0; sl < NSL; sl++) { vh[sl] = ldg16(pj.vhi + at + sl * 16); vl[sl] = ldg16(pj.vlo + at + sl * 16); }
        };
        // up to four tiles (s_list[base .. base + nrun)): request their B rows, then apply them
        auto flush = [&](int base, int count, int nrun, bool first) {
            int i0[4], i1[4];
            __syncthreads();                       // the stages and the tables are free (main loop or previous batch done)
            if (!first) {
                fill_rows(base, count);
                __syncthreads();
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                i0[q] = __builtin_amdgcn_readfirstlane(s_span[q][0]);    // rows of the block, may stick out on either side
                i1[q] = __builtin_amdgcn_readfirstlane(s_span[q][1]);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (q >= nrun) continue;
                unsigned char *stage = q == 0 ? smem : q == 1 ? smem1 : q == 2 ? smem2 : smem3;
                const unsigned lbase = (unsigned)(__UINTPTR_TYPE__)(lds_byte *)stage + (unsigned)wave * 1024u;
#pragma unroll
                for (int u = 0; u < RMAX / 8; u++) b_rows_load(b_row_of(q, u), u, lbase);
            }
            uint4 vh[2][NSL], vl[2][NSL];
            load_v(0, vh[0], vl[0]);
            GL_WAIT_LOADS(0);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (i + 1 < 4) load_v(i + 1, vh[(i + 1) & 1], vl[(i + 1) & 1]);
                const int R0 = wm * 128 + i * 32, my = R0 + l32;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (q >= nrun || R0 + 32 <= i0[q] || R0 >= i1[q]) continue;       // uniform per wavefront
                    const unsigned char *stage = q == 0 ? smem : q == 1 ? smem1 : q == 2 ? smem2 : smem3;
                    const unsigned keep = (my >= i0[q] && my < i1[q]) ? 0xffffffffu : 0u;
                    uint4 bf[2][4];                 // W-side operands, one slice ahead
                    w_frags(stage, 0, bf[0]);
#pragma unroll
                    for (int sl = 0; sl < NSL; sl++) {
                        if (sl + 1 < NSL) w_frags(stage, sl + 1, bf[(sl + 1) & 1]);
                        const uint4 h = vh[i & 1][sl], l = vl[i & 1][sl];
                        const uint4 xh = make_uint4(h.x & keep, h.y & keep, h.z & keep, h.w & keep);
                        const uint4 xl = make_uint4(l.x & keep, l.y & keep, l.z & keep, l.w & keep);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            acc[i][j] = mfma32<DT>(xh, bf[sl & 1][j], acc[i][j]);
                            acc[i][j] = mfma32<DT>(xl, bf[sl & 1][j], acc[i][j]);
                        }
                    }
                }
            }
        };
#pragma unroll 1
        for (int b0 = 0; b0 < n_plan; b0 += G_NT) {
            if (b0 > 0) list_tiles(b0);            // the first 256 tiles were looked at before the K loop
            const int count = __builtin_amdgcn_readfirstlane(s_list[G_NT]);
#pragma unroll 1
            for (int base = 0; base < count; base += 4)
                flush(base, count, count - base < 4 ? count - base : 4, b0 == 0 && base == 0);
            __syncthreads();                       // s_list is free for the next 256 tiles
        }
        __syncthreads();
    }
#undef GL_WAIT_LOADS

    // ---- y: every wavefront passes its 128 x 128 block through a private LDS tile, 32 rows at a time, so
    // that the stores are 16 bytes wide and a 16-lane row covers 256 contiguous bytes of one token.
    // D layout of the 32x32 MFMA: lane holds column lane % 32, rows 8 * (e / 4) + 4 * (lane / 32) + e % 4.
    // The tile is private to the wavefront and LDS operations of one wavefront complete in order, so no
    // barrier is needed; the accesses are volatile so that they stay in program order.
    {
        unsigned char *so = wave == 0 ? smem : wave == 1 ? smem1 : wave == 2 ? smem2 : smem3;
        typedef __attribute__((address_space(3))) volatile uint16_t lds_vu16;
        typedef __attribute__((address_space(3))) volatile u32x4_t lds_vu32x4;
        uint16_t *__restrict__ y = static_cast<uint16_t *>(pj.y);
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int e = 0; e < 16; e += 2) {
                    // two rows of one column, converted as a pair by the hardware (round to nearest even)
                    const uint32_t u = pack2<DT>(acc[i][j][e], acc[i][j][e + 1]);
                    const int row = 8 * (e >> 2) + 4 * lh + (e & 3);
                    *(lds_vu16 *)(so + row * OPITCH + (j * 32 + l32) * 2) = (uint16_t)u;
                    *(lds_vu16 *)(so + (row + 1) * OPITCH + (j * 32 + l32) * 2) = (uint16_t)(u >> 16);
                }
#pragma unroll
            for (int q = 0; q < 8; q++) {
                const int pp = lane + 64 * q, row = pp >> 4, c = pp & 15;
                const u32x4_t v = *(lds_vu32x4 *)(so + row * OPITCH + c * 16);
                const int gr = m0 + wm * 128 + i * 32 + row, gc = n0 + wn * 128 + c * 8;
                if (gr < T && gc < hout) stg16_stream(y + (size_t)gr * hout + gc, make_uint4(v.x, v.y, v.z, v.w));
            }
        }
    }
}

template <int DT, int RMAX>
static int launch_gl(const GemmLoraArgs &a, hipStream_t s)
{
    GemmLoraArgs g = a;
    g.rmax = RMAX;
    g.ntm = (g.T + GM - 1) / GM;
    // projections with the longest K loop first: their tiles take longest, and a long tile started last
    // would leave the rest of the device idle at the end of the launch
    for (int q = 1; q < g.n_proj; q++)
        for (int r = q; r > 0 && g.pr[r].hin > g.pr[r - 1].hin; r--) {
            const GemmProj t = g.pr[r]; g.pr[r] = g.pr[r - 1]; g.pr[r - 1] = t;
        }
    unsigned end = 0;
    for (int q = 0; q < g.n_proj; q++) {
        g.pr[q].ntn = (g.pr[q].hout + GN - 1) / GN;
        const long long tiles = (long long)g.ntm * g.pr[q].ntn;
        const long long padded = (tiles + 7) / 8 * 8;
        if (end + padded > 0x7fffffffLL) return (int)hipErrorInvalidValue;
        end += (unsigned)padded;
        g.pr[q].end = end;
    }
    if (end == 0) return 0;
    if (g.lora) {
        hipLaunchKernelGGL((gemm_lora_reduce_kernel<DT, RMAX>), dim3((unsigned)g.max_tiles, (unsigned)g.n_proj), dim3(256), 0, s, g);
        const int rc = (int)hipGetLastError();
        if (rc) return rc;
    }
    hipLaunchKernelGGL((gemm_lora_kernel<DT, RMAX>), dim3(end), dim3(G_NT), 0, s, g);
    return (int)hipGetLastError();
}

int launch_gemm_lora(const GemmLoraArgs &a, int dtype, int max_rank, hipStream_t s)
{
    if (dtype == DT_F16) {
        if (max_rank <= 16) return launch_gl<DT_F16, 16>(a, s);
        if (max_rank <= 32) return launch_gl<DT_F16, 32>(a, s);
        return launch_gl<DT_F16, 64>(a, s);
    }
    if (max_rank <= 16) return launch_gl<DT_BF16, 16>(a, s);
    if (max_rank <= 32) return launch_gl<DT_BF16, 32>(a, s);
    return launch_gl<DT_BF16, 64>(a, s);
}

}  // namespace mlora
