// libmlora_cpu.so: the CPU side of the CPU-assisted LoRA path (declared in include/mlora_cpu.h).
//
//   - the worker arithmetic of lora_cpu/lora_shm_op/app.py:136-141 (res = x.float() @ down @ up; half)
//     on AVX2 + F16C, a few tokens at a time so that an adapter's weights are read once per token block;
//   - a batch entry point that cuts the tokens into tasks the way the reference shards a request over its
//     workers (lightllm/models/lora_cpu.py:150-151) and runs them on a persistent thread pool;
//   - the polling loop of the workers (app.py:102-143) over the transport's request slots, result slots
//     and signal table, as one in-process thread that hands the chunks to the same pool.
//
// Summation order is fixed (ascending column index in the down projection, ascending rank index in the
// up projection, multiply and add as separate roundings), so a token's result is the same bits whatever
// the task cut, the token-block position or the thread count.
#include <immintrin.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <thread>
#include <vector>

#include "../../../include/mlora_cpu.h"
#include "task_pool.hpp"

namespace {

using mlora_cpu::TaskPool;

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

constexpr int TB = 4;   // tokens that share one pass over an adapter's weights

// ---------------------------------------------------------------- 16-bit rows
inline void row_f16_to_f32(const uint16_t *src, float *dst, int n)
{
    int i = 0;
    for (; i + 8 <= n; i += 8)
        _mm256_storeu_ps(dst + i, _mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(src + i))));
    if (i < n) {
        uint16_t tail[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        float out[8];
        memcpy(tail, src + i, (size_t)(n - i) * 2);
        _mm256_storeu_ps(out, _mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(tail))));
        memcpy(dst + i, out, (size_t)(n - i) * 4);
    }
}

// 8 weights starting at element `at` of a row that ends at element `end` (lanes beyond the row read as zero)
template <bool W16>
inline __m256 load_w8(const void *base, size_t at, size_t end)
{
    if (at + 8 <= end) {
        if constexpr (W16)
            return _mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(static_cast<const uint16_t *>(base) + at)));
        else
            return _mm256_loadu_ps(static_cast<const float *>(base) + at);
    }
    const size_t n = end > at ? end - at : 0;
    if constexpr (W16) {
        uint16_t tail[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        memcpy(tail, static_cast<const uint16_t *>(base) + at, n * 2);
        return _mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(tail)));
    } else {
        float tail[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        memcpy(tail, static_cast<const float *>(base) + at, n * 4);
        return _mm256_loadu_ps(tail);
    }
}

// ---------------------------------------------------------------- down projection
// v[t][j] = sum_k x[t][k] * down[k][j], k ascending, for up to TB tokens; RV vectors of 8 ranks held in
// registers (RV * TB <= 8 accumulators), or any rank through memory when RV == 0.
template <bool W16, int RV, int NT>
void shrink_fixed(const float *xf, int Hin, const void *down, int r, float *v, int rp)
{
    __m256 acc[NT][RV];
    for (int t = 0; t < NT; t++)
        for (int q = 0; q < RV; q++) acc[t][q] = _mm256_setzero_ps();
    for (int k = 0; k < Hin; k++) {
        const size_t row0 = (size_t)k * r;
        __m256 d[RV];
        for (int q = 0; q < RV; q++) d[q] = load_w8<W16>(down, row0 + 8 * q, row0 + r);
        for (int t = 0; t < NT; t++) {
            const __m256 xv = _mm256_set1_ps(xf[(size_t)t * Hin + k]);
            for (int q = 0; q < RV; q++) acc[t][q] = _mm256_add_ps(acc[t][q], _mm256_mul_ps(xv, d[q]));
        }
    }
    for (int t = 0; t < NT; t++)
        for (int q = 0; q < RV; q++) _mm256_storeu_ps(v + (size_t)t * rp + 8 * q, acc[t][q]);
}

template <bool W16>
void shrink_any(const float *xf, int nt, int Hin, const void *down, int r, float *v, int rp)
{
    const int rv = rp / 8;
    for (int t = 0; t < nt; t++)
        for (int j = 0; j < rp; j++) v[(size_t)t * rp + j] = 0.f;
    for (int k = 0; k < Hin; k++) {
        const size_t row0 = (size_t)k * r;
        for (int q = 0; q < rv; q++) {
            const __m256 d = load_w8<W16>(down, row0 + 8 * q, row0 + r);
            for (int t = 0; t < nt; t++) {
                float *a = v + (size_t)t * rp + 8 * q;
                const __m256 xv = _mm256_set1_ps(xf[(size_t)t * Hin + k]);
                _mm256_storeu_ps(a, _mm256_add_ps(_mm256_loadu_ps(a), _mm256_mul_ps(xv, d)));
            }
        }
    }
}

template <bool W16>
void shrink(const float *xf, int nt, int Hin, const void *down, int r, float *v, int rp)
{
    const int rv = rp / 8;
    if (nt == TB && rv == 1) return shrink_fixed<W16, 1, TB>(xf, Hin, down, r, v, rp);
    if (nt == TB && rv == 2) return shrink_fixed<W16, 2, TB>(xf, Hin, down, r, v, rp);
    if (nt >= 2 && rv == 4) {
        for (int t = 0; t + 2 <= nt; t += 2) shrink_fixed<W16, 4, 2>(xf + (size_t)t * Hin, Hin, down, r, v + (size_t)t * rp, rp);
        if (nt & 1) shrink_fixed<W16, 4, 1>(xf + (size_t)(nt - 1) * Hin, Hin, down, r, v + (size_t)(nt - 1) * rp, rp);
        return;
    }
    if (rv == 8) {
        for (int t = 0; t < nt; t++) shrink_fixed<W16, 8, 1>(xf + (size_t)t * Hin, Hin, down, r, v + (size_t)t * rp, rp);
        return;
    }
    if (rv == 1) { for (int t = 0; t < nt; t++) shrink_fixed<W16, 1, 1>(xf + (size_t)t * Hin, Hin, down, r, v + (size_t)t * rp, rp); return; }
    if (rv == 2) { for (int t = 0; t < nt; t++) shrink_fixed<W16, 2, 1>(xf + (size_t)t * Hin, Hin, down, r, v + (size_t)t * rp, rp); return; }
    if (rv == 4) return shrink_fixed<W16, 4, 1>(xf, Hin, down, r, v, rp);
    shrink_any<W16>(xf, nt, Hin, down, r, v, rp);
}

// ---------------------------------------------------------------- up projection
// out[t][c] = half( y0[t][c] + scale * sum_j v[t][j] * up[j][c] ), j ascending; 16 columns x NT tokens per step.
template <bool W16, int NT>
void expand_fixed(const float *v, int rp, const void *up, int r, int Hout, float scale, const uint16_t *y0, uint16_t *y)
{
    const __m256 sc = _mm256_set1_ps(scale);
    int c = 0;
    for (; c + 16 <= Hout; c += 16) {
        __m256 a0[NT], a1[NT];
        for (int t = 0; t < NT; t++) { a0[t] = _mm256_setzero_ps(); a1[t] = _mm256_setzero_ps(); }
        for (int j = 0; j < r; j++) {
            const size_t at = (size_t)j * Hout + c;
            const __m256 u0 = load_w8<W16>(up, at, at + 8), u1 = load_w8<W16>(up, at + 8, at + 16);
            for (int t = 0; t < NT; t++) {
                const __m256 vj = _mm256_set1_ps(v[(size_t)t * rp + j]);
                a0[t] = _mm256_add_ps(a0[t], _mm256_mul_ps(vj, u0));
                a1[t] = _mm256_add_ps(a1[t], _mm256_mul_ps(vj, u1));
            }
        }
        for (int t = 0; t < NT; t++) {
            __m256 r0 = a0[t], r1 = a1[t];
            if (scale != 1.0f) { r0 = _mm256_mul_ps(r0, sc); r1 = _mm256_mul_ps(r1, sc); }
            if (y0) {
                const uint16_t *b = y0 + (size_t)t * Hout + c;
                r0 = _mm256_add_ps(_mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(b))), r0);
                r1 = _mm256_add_ps(_mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(b + 8))), r1);
            }
            uint16_t *o = y + (size_t)t * Hout + c;
            _mm_storeu_si128(reinterpret_cast<__m128i *>(o), _mm256_cvtps_ph(r0, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
            _mm_storeu_si128(reinterpret_cast<__m128i *>(o + 8), _mm256_cvtps_ph(r1, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
        }
    }
    // column tail: 8 at a time through a padded buffer, same order of operations
    for (; c < Hout; c += 8) {
        const int n = Hout - c < 8 ? Hout - c : 8;
        for (int t = 0; t < NT; t++) {
            __m256 a = _mm256_setzero_ps();
            for (int j = 0; j < r; j++) {
                const size_t at = (size_t)j * Hout + c;
                a = _mm256_add_ps(a, _mm256_mul_ps(_mm256_set1_ps(v[(size_t)t * rp + j]), load_w8<W16>(up, at, at + n)));
            }
            if (scale != 1.0f) a = _mm256_mul_ps(a, sc);
            if (y0) {
                uint16_t b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                memcpy(b, y0 + (size_t)t * Hout + c, (size_t)n * 2);
                a = _mm256_add_ps(_mm256_cvtph_ps(_mm_loadu_si128(reinterpret_cast<const __m128i *>(b))), a);
            }
            uint16_t o[8];
            _mm_storeu_si128(reinterpret_cast<__m128i *>(o), _mm256_cvtps_ph(a, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
            memcpy(y + (size_t)t * Hout + c, o, (size_t)n * 2);
        }
    }
}

template <bool W16>
void expand(const float *v, int nt, int rp, const void *up, int r, int Hout, float scale, const uint16_t *y0, uint16_t *y)
{
    switch (nt) {
    case 4: return expand_fixed<W16, 4>(v, rp, up, r, Hout, scale, y0, y);
    case 3: return expand_fixed<W16, 3>(v, rp, up, r, Hout, scale, y0, y);
    case 2: return expand_fixed<W16, 2>(v, rp, up, r, Hout, scale, y0, y);
    default: return expand_fixed<W16, 1>(v, rp, up, r, Hout, scale, y0, y);
    }
}

struct Scratch {
    std::vector<float> xf, v;
};

// n_tok consecutive tokens through one adapter's weights (down [Hin, r], up [r, Hout]).
template <bool W16>
void lora_tokens(const uint16_t *x, const void *down, const void *up, const uint16_t *y0, uint16_t *y,
                 int n_tok, int Hin, int Hout, int r, float scale)
{
    thread_local Scratch s;
    const int rp = (r + 7) / 8 * 8;
    if (s.xf.size() < (size_t)TB * Hin) s.xf.resize((size_t)TB * Hin);
    if (s.v.size() < (size_t)TB * rp) s.v.resize((size_t)TB * rp);
    for (int t0 = 0; t0 < n_tok; t0 += TB) {
        const int nt = n_tok - t0 < TB ? n_tok - t0 : TB;
        for (int t = 0; t < nt; t++) row_f16_to_f32(x + (size_t)(t0 + t) * Hin, s.xf.data() + (size_t)t * Hin, Hin);
        shrink<W16>(s.xf.data(), nt, Hin, down, r, s.v.data(), rp);
        expand<W16>(s.v.data(), nt, rp, up, r, Hout, scale, y0 ? y0 + (size_t)t0 * Hout : nullptr, y + (size_t)t0 * Hout);
    }
}

void lora_tokens_dt(int w_dtype, const uint16_t *x, const void *down, const void *up, const uint16_t *y0, uint16_t *y,
                    int n_tok, int Hin, int Hout, int r, float scale)
{
    if (w_dtype == MLORA_CPU_W_F16) lora_tokens<true>(x, down, up, y0, y, n_tok, Hin, Hout, r, scale);
    else lora_tokens<false>(x, down, up, y0, y, n_tok, Hin, Hout, r, scale);
}

inline const void *adapter_weights(const void *base, int w_dtype, int adapter, size_t elems)
{
    const size_t bytes = elems * (w_dtype == MLORA_CPU_W_F16 ? 2u : 4u);
    return static_cast<const unsigned char *>(base) + (size_t)adapter * bytes;
}

struct Task { int tok0, n, adapter; };

// ---------------------------------------------------------------- in-process workers of the transport
struct AssistServer {
    TaskPool *pool;
    const uint16_t *x_slots;
    uint16_t *out_slots[MLORA_CPU_ASSIST_MAX_PROJ];
    int16_t *signals;
    const int32_t *tkn_len;
    int n_proj, n_workers, n_slots, slot_tokens, H, cap;
    const void *down[MLORA_CPU_ASSIST_MAX_PROJ];
    const void *up[MLORA_CPU_ASSIST_MAX_PROJ];
    int w_dtype, r, n_adapters;
    const int32_t *slot_adapter;
    int sig_base, sig_stride;
    std::vector<std::atomic<int>> busy;        // [n_proj * n_workers]: a chunk of this worker is queued or running
    std::atomic<int> in_flight{0};
    std::atomic<bool> stop{false};
    std::atomic<int64_t> served{0}, rejected{0};
    std::thread poller;

    AssistServer(int n) : busy((size_t)n) {}

    void clear_signal(int q, int w) { __atomic_store_n(&signals[(size_t)q * n_workers + w], (int16_t)0, __ATOMIC_RELEASE); }

    void chunk(int q, int w, int req, int tok0, int ntok)
    {
        const int a = slot_adapter ? slot_adapter[req] : 0;
        const size_t at = ((size_t)req * slot_tokens + tok0) * H;
        lora_tokens_dt(w_dtype, x_slots + at, adapter_weights(down[q], w_dtype, a, (size_t)H * r),
                       adapter_weights(up[q], w_dtype, a, (size_t)r * H), nullptr, out_slots[q] + at, ntok, H, H, r, 1.0f);
        served.fetch_add(1, std::memory_order_relaxed);
        clear_signal(q, w);                    // results first, then the worker's "done" (release store)
        busy[(size_t)q * n_workers + w].store(0, std::memory_order_release);
        in_flight.fetch_sub(1, std::memory_order_release);
    }

    void poll()
    {
        unsigned idle = 0;
        while (!stop.load(std::memory_order_acquire)) {
            bool any = false;
            for (int q = 0; q < n_proj; q++) {
                for (int w = 0; w < n_workers; w++) {
                    // busy first, the code after it: a chunk clears its signal before it drops `busy`, so a
                    // code read after seeing busy == 0 is never the one that chunk has just served
                    std::atomic<int> &b = busy[(size_t)q * n_workers + w];
                    if (b.load(std::memory_order_acquire)) continue;
                    const int code = __atomic_load_n(&signals[(size_t)q * n_workers + w], __ATOMIC_ACQUIRE);
                    if (code <= 1) continue;
                    any = true;
                    // the code names the projection and the row (app.py:110-128); it must belong to this cell
                    const int row = code - sig_base - q * sig_stride;
                    const int tkn = __atomic_load_n(tkn_len, __ATOMIC_ACQUIRE);
                    bool ok = row == w && tkn > 0 && tkn <= slot_tokens;
                    int req = 0, tok0 = 0, ntok = 0;
                    if (ok) {
                        const int cpr = (tkn - 1) / cap + 1;
                        req = row / cpr;
                        tok0 = (row % cpr) * cap;
                        ntok = (tok0 + cap < tkn ? tok0 + cap : tkn) - tok0;
                        ok = req < n_slots && ntok > 0;
                        if (ok && slot_adapter) ok = slot_adapter[req] >= 0 && slot_adapter[req] < n_adapters;
                    }
                    if (!ok) {
                        rejected.fetch_add(1, std::memory_order_relaxed);
                        clear_signal(q, w);
                        continue;
                    }
                    b.store(1, std::memory_order_release);
                    in_flight.fetch_add(1, std::memory_order_acq_rel);
                    pool->submit(1, [this, q, w, req, tok0, ntok](int) { chunk(q, w, req, tok0, ntok); });
                }
            }
            if (any) idle = 0;
            else if (++idle < 2000) _mm_pause();
            else std::this_thread::yield();
        }
        while (in_flight.load(std::memory_order_acquire) > 0) std::this_thread::yield();
    }
};

}  // namespace

extern "C" {

const char *mlora_cpu_last_error(void) { return g_err; }
int mlora_cpu_version(void) { return 100; }

void *mlora_cpu_pool_create(int n_threads)
{
    if (n_threads < 1 || n_threads > MLORA_CPU_MAX_THREADS) {
        fail(MLORA_CPU_ERANGE, "n_threads must be in 1..%d (got %d)", MLORA_CPU_MAX_THREADS, n_threads);
        return nullptr;
    }
    return new TaskPool(n_threads);
}

void mlora_cpu_pool_destroy(void *pool) { delete static_cast<TaskPool *>(pool); }

int mlora_cpu_pool_threads(void *pool) { return pool ? static_cast<TaskPool *>(pool)->threads() : 0; }

int mlora_cpu_lora(void *pool, const uint16_t *x, const void *A, const void *B, int w_dtype,
                   const int32_t *tok_adapter, const uint16_t *y0, uint16_t *y,
                   int T, int Hin, int Hout, int r, int n_adapters, float scale, int tokens_per_task)
{
    if (T < 0) return fail(MLORA_CPU_EINVAL, "T must be >= 0 (got %d)", T);
    if (T == 0) return MLORA_CPU_OK;
    if (!x || !A || !B || !tok_adapter || !y) return fail(MLORA_CPU_EINVAL, "NULL pointer");
    if (Hin <= 0 || Hout <= 0) return fail(MLORA_CPU_EINVAL, "Hin and Hout must be positive (got %d, %d)", Hin, Hout);
    if (r < 1 || r > MLORA_CPU_MAX_RANK) return fail(MLORA_CPU_ERANGE, "rank must be in 1..%d (got %d)", MLORA_CPU_MAX_RANK, r);
    if (n_adapters < 1) return fail(MLORA_CPU_EINVAL, "n_adapters must be positive (got %d)", n_adapters);
    if (w_dtype != MLORA_CPU_W_F32 && w_dtype != MLORA_CPU_W_F16) return fail(MLORA_CPU_EINVAL, "w_dtype must be MLORA_CPU_W_F32 or MLORA_CPU_W_F16 (got %d)", w_dtype);
    if (tokens_per_task < 1) return fail(MLORA_CPU_EINVAL, "tokens_per_task must be positive (got %d)", tokens_per_task);
    for (int t = 0; t < T; t++)
        if (tok_adapter[t] >= n_adapters) return fail(MLORA_CPU_ERANGE, "token %d names adapter %d of %d", t, tok_adapter[t], n_adapters);

    std::vector<Task> tasks;
    for (int t = 0; t < T;) {
        const int a = tok_adapter[t];
        int e = t + 1;
        while (e < T && e - t < tokens_per_task && tok_adapter[e] == a) e++;
        tasks.push_back(Task{t, e - t, a});
        t = e;
    }
    auto one = [&](int i) {
        const Task &k = tasks[(size_t)i];
        uint16_t *out = y + (size_t)k.tok0 * Hout;
        if (k.adapter < 0) {
            if (y0) memcpy(out, y0 + (size_t)k.tok0 * Hout, (size_t)k.n * Hout * 2);
            else memset(out, 0, (size_t)k.n * Hout * 2);
            return;
        }
        lora_tokens_dt(w_dtype, x + (size_t)k.tok0 * Hin, adapter_weights(A, w_dtype, k.adapter, (size_t)Hin * r),
                       adapter_weights(B, w_dtype, k.adapter, (size_t)r * Hout), y0 ? y0 + (size_t)k.tok0 * Hout : nullptr,
                       out, k.n, Hin, Hout, r, scale);
    };
    if (pool) static_cast<TaskPool *>(pool)->run((int)tasks.size(), one);
    else for (int i = 0; i < (int)tasks.size(); i++) one(i);
    return MLORA_CPU_OK;
}

void *mlora_cpu_assist_start(void *pool, const uint16_t *x_slots, uint16_t *const *out_slots, int16_t *signals,
                             const int32_t *tkn_len, int n_proj, int n_workers, int n_slots, int slot_tokens, int H,
                             int cap, const void *const *down, const void *const *up, int w_dtype, int r, int n_adapters,
                             const int32_t *slot_adapter, int sig_base, int sig_stride)
{
    if (!pool) { fail(MLORA_CPU_ESTATE, "a worker pool is needed"); return nullptr; }
    if (!x_slots || !out_slots || !signals || !tkn_len || !down || !up) { fail(MLORA_CPU_EINVAL, "NULL pointer"); return nullptr; }
    if (n_proj < 1 || n_proj > MLORA_CPU_ASSIST_MAX_PROJ) { fail(MLORA_CPU_ERANGE, "n_proj must be in 1..%d (got %d)", MLORA_CPU_ASSIST_MAX_PROJ, n_proj); return nullptr; }
    if (n_workers < 1 || n_slots < 1 || slot_tokens < 1 || H < 1 || cap < 1 || n_adapters < 1) { fail(MLORA_CPU_EINVAL, "sizes must be positive"); return nullptr; }
    if (r < 1 || r > MLORA_CPU_MAX_RANK) { fail(MLORA_CPU_ERANGE, "rank must be in 1..%d (got %d)", MLORA_CPU_MAX_RANK, r); return nullptr; }
    if (w_dtype != MLORA_CPU_W_F32 && w_dtype != MLORA_CPU_W_F16) { fail(MLORA_CPU_EINVAL, "bad w_dtype %d", w_dtype); return nullptr; }
    if (sig_base < 2 || sig_stride < n_workers || (long long)sig_base + (long long)sig_stride * n_proj > 32767) {
        fail(MLORA_CPU_ERANGE, "signal codes must be > 1, distinct per projection and fit 16 bits");
        return nullptr;
    }
    for (int q = 0; q < n_proj; q++)
        if (!out_slots[q] || !down[q] || !up[q]) { fail(MLORA_CPU_EINVAL, "projection %d: NULL pointer", q); return nullptr; }
    AssistServer *s = new AssistServer(n_proj * n_workers);
    s->pool = static_cast<TaskPool *>(pool);
    s->x_slots = x_slots; s->signals = signals; s->tkn_len = tkn_len;
    for (int q = 0; q < n_proj; q++) { s->out_slots[q] = out_slots[q]; s->down[q] = down[q]; s->up[q] = up[q]; }
    s->n_proj = n_proj; s->n_workers = n_workers; s->n_slots = n_slots; s->slot_tokens = slot_tokens; s->H = H; s->cap = cap;
    s->w_dtype = w_dtype; s->r = r; s->n_adapters = n_adapters; s->slot_adapter = slot_adapter;
    s->sig_base = sig_base; s->sig_stride = sig_stride;
    for (auto &b : s->busy) b.store(0);
    s->poller = std::thread([s] { s->poll(); });
    return s;
}

int mlora_cpu_assist_stop(void *server, int64_t *served, int64_t *rejected)
{
    if (!server) return fail(MLORA_CPU_ESTATE, "NULL server handle");
    AssistServer *s = static_cast<AssistServer *>(server);
    s->stop.store(true, std::memory_order_release);
    s->poller.join();
    if (served) *served = s->served.load();
    if (rejected) *rejected = s->rejected.load();
    delete s;
    return MLORA_CPU_OK;
}

}  // extern "C"
