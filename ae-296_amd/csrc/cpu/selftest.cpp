// Self-test driver for libmlora_cpu's sources, built with AddressSanitizer + UBSan and with ThreadSanitizer
// (see Makefile) and run by tests/test_cpu_lora.py.  Exercises: the pool under many small batches submitted
// from several threads; mlora_cpu_lora on ragged sizes (rank and width tails) against a scalar restatement
// in the same summation order (bit for bit), single-threaded against pooled; the transport's in-process
// workers with this program playing the GPU side (writes the request slots, raises the codes, waits for the
// signals to drop), including codes that must be rejected.  Exit code 0 = all good.
#include <immintrin.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#include "../../../include/mlora_cpu.h"
#include "task_pool.hpp"

static int g_failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { g_failures++; fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); fprintf(stderr, __VA_ARGS__); fprintf(stderr, "\n"); } } while (0)

static float h2f(uint16_t h) { return _cvtsh_ss(h); }
static uint16_t f2h(float f) { return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC); }

// volatile stores keep the compiler from contracting or reassociating the scalar restatement
static void scalar_lora(const uint16_t *x, const float *down, const float *up, const uint16_t *y0, uint16_t *y,
                        int Hin, int Hout, int r, float scale)
{
    std::vector<float> v((size_t)r, 0.f);
    for (int k = 0; k < Hin; k++)
        for (int j = 0; j < r; j++) { volatile float p = h2f(x[k]) * down[(size_t)k * r + j]; v[(size_t)j] = v[(size_t)j] + p; }
    for (int c = 0; c < Hout; c++) {
        float acc = 0.f;
        for (int j = 0; j < r; j++) { volatile float p = v[(size_t)j] * up[(size_t)j * Hout + c]; acc = acc + p; }
        if (scale != 1.0f) { volatile float s = acc * scale; acc = s; }
        if (y0) acc = h2f(y0[c]) + acc;
        y[c] = f2h(acc);
    }
}

static void test_pool()
{
    mlora_cpu::TaskPool pool(4);
    std::atomic<long> sum{0};
    std::vector<std::thread> subs;
    for (int s = 0; s < 3; s++)
        subs.emplace_back([&pool, &sum, s] {
            for (int rep = 0; rep < 200; rep++) {
                const int n = 1 + (rep * 7 + s) % 13;
                pool.run(n, [&sum](int i) { sum.fetch_add(i + 1, std::memory_order_relaxed); });
            }
        });
    for (auto &t : subs) t.join();
    long want = 0;
    for (int s = 0; s < 3; s++)
        for (int rep = 0; rep < 200; rep++) { const int n = 1 + (rep * 7 + s) % 13; want += (long)n * (n + 1) / 2; }
    CHECK(sum.load() == want, "pool ran %ld, expected %ld", sum.load(), want);
    auto b = pool.submit(0, [](int) {});
    b->wait();
    CHECK(b->done(), "empty batch not done");
}

static void test_lora(int T, int Hin, int Hout, int r, int N, int threads, int per_task, bool with_y0, float scale, unsigned seed)
{
    std::mt19937 rng(seed);
    std::normal_distribution<float> nd(0.f, 1.f);
    std::vector<uint16_t> x((size_t)T * Hin), y0((size_t)T * Hout), y((size_t)T * Hout, 0x7e00), y1((size_t)T * Hout, 0x7e00), want((size_t)T * Hout);
    std::vector<float> A((size_t)N * Hin * r), B((size_t)N * r * Hout);
    std::vector<int32_t> tok((size_t)T);
    for (auto &e : x) e = f2h(nd(rng));
    for (auto &e : y0) e = f2h(nd(rng));
    for (auto &e : A) e = 0.05f * nd(rng);
    for (auto &e : B) e = 0.05f * nd(rng);
    for (auto &e : tok) e = (int)(rng() % (unsigned)(N + 1)) - 1;
    for (int t = 0; t < T; t++) {
        const int a = tok[(size_t)t];
        uint16_t *w = want.data() + (size_t)t * Hout;
        if (a < 0) { for (int c = 0; c < Hout; c++) w[c] = with_y0 ? y0[(size_t)t * Hout + c] : 0; continue; }
        scalar_lora(x.data() + (size_t)t * Hin, A.data() + (size_t)a * Hin * r, B.data() + (size_t)a * r * Hout,
                    with_y0 ? y0.data() + (size_t)t * Hout : nullptr, w, Hin, Hout, r, scale);
    }
    void *pool = mlora_cpu_pool_create(threads);
    CHECK(pool && mlora_cpu_pool_threads(pool) == threads, "pool create");
    int rc = mlora_cpu_lora(pool, x.data(), A.data(), B.data(), MLORA_CPU_W_F32, tok.data(), with_y0 ? y0.data() : nullptr, y.data(),
                            T, Hin, Hout, r, N, scale, per_task);
    CHECK(rc == 0, "mlora_cpu_lora rc %d: %s", rc, mlora_cpu_last_error());
    CHECK(memcmp(y.data(), want.data(), y.size() * 2) == 0, "pooled result differs from the scalar restatement (T=%d Hin=%d Hout=%d r=%d)", T, Hin, Hout, r);
    rc = mlora_cpu_lora(nullptr, x.data(), A.data(), B.data(), MLORA_CPU_W_F32, tok.data(), with_y0 ? y0.data() : nullptr, y1.data(),
                        T, Hin, Hout, r, N, scale, 1);
    CHECK(rc == 0 && memcmp(y1.data(), want.data(), y1.size() * 2) == 0, "inline one-token tasks differ (T=%d r=%d)", T, r);
    // binary16 weights: the same values when the fp32 weights are representable
    std::vector<uint16_t> A16(A.size()), B16(B.size());
    std::vector<float> Ar(A.size()), Br(B.size());
    for (size_t i = 0; i < A.size(); i++) { A16[i] = f2h(A[i]); Ar[i] = h2f(A16[i]); }
    for (size_t i = 0; i < B.size(); i++) { B16[i] = f2h(B[i]); Br[i] = h2f(B16[i]); }
    rc = mlora_cpu_lora(pool, x.data(), A16.data(), B16.data(), MLORA_CPU_W_F16, tok.data(), nullptr, y.data(), T, Hin, Hout, r, N, 1.0f, per_task);
    int rc2 = mlora_cpu_lora(pool, x.data(), Ar.data(), Br.data(), MLORA_CPU_W_F32, tok.data(), nullptr, y1.data(), T, Hin, Hout, r, N, 1.0f, per_task);
    CHECK(rc == 0 && rc2 == 0 && memcmp(y.data(), y1.data(), y.size() * 2) == 0, "binary16 weights differ from their fp32 values (r=%d)", r);
    tok[0] = N;
    rc = mlora_cpu_lora(pool, x.data(), A.data(), B.data(), MLORA_CPU_W_F32, tok.data(), nullptr, y.data(), T, Hin, Hout, r, N, 1.0f, per_task);
    CHECK(rc == MLORA_CPU_ERANGE, "adapter id beyond the pool accepted (rc %d)", rc);
    mlora_cpu_pool_destroy(pool);
}

static void test_assist()
{
    const int n_proj = 3, n_workers = 6, n_slots = 4, slot_tokens = 16, H = 40, cap = 5, r = 12, N = 2, base = 2, stride = 200;
    std::mt19937 rng(99);
    std::normal_distribution<float> nd(0.f, 1.f);
    std::vector<uint16_t> xs((size_t)n_slots * slot_tokens * H, 0);
    std::vector<std::vector<uint16_t>> outs(n_proj, std::vector<uint16_t>((size_t)n_slots * slot_tokens * H, 0xdead));
    std::vector<std::vector<float>> down(n_proj, std::vector<float>((size_t)N * H * r)), up(n_proj, std::vector<float>((size_t)N * r * H));
    for (auto &d : down) for (auto &e : d) e = 0.1f * nd(rng);
    for (auto &u : up) for (auto &e : u) e = 0.1f * nd(rng);
    std::vector<int16_t> sig((size_t)n_proj * n_workers, 0);
    int32_t tkn_len = 0;
    const int32_t slot_adapter[n_slots] = {1, 0, 1, 0};
    uint16_t *op[n_proj];
    const void *dp[n_proj], *upp[n_proj];
    for (int q = 0; q < n_proj; q++) { op[q] = outs[(size_t)q].data(); dp[q] = down[(size_t)q].data(); upp[q] = up[(size_t)q].data(); }
    void *pool = mlora_cpu_pool_create(3);
    void *srv = mlora_cpu_assist_start(pool, xs.data(), op, sig.data(), &tkn_len, n_proj, n_workers, n_slots, slot_tokens, H, cap,
                                       dp, upp, MLORA_CPU_W_F32, r, N, slot_adapter, base, stride);
    CHECK(srv != nullptr, "assist start: %s", mlora_cpu_last_error());
    if (!srv) { mlora_cpu_pool_destroy(pool); return; }
    long served_want = 0;
    for (int round = 0; round < 3; round++) {
        const int batch = 2, tkn = 7 + round * 2;                     // cpr = 2, 2, 3 -> 4, 4, 6 workers
        const int cpr = (tkn - 1) / cap + 1, active = batch * cpr;
        for (int b = 0; b < batch; b++)
            for (int t = 0; t < tkn; t++)
                for (int c = 0; c < H; c++) xs[((size_t)b * slot_tokens + t) * H + c] = f2h(nd(rng));
        __atomic_store_n(&tkn_len, tkn, __ATOMIC_RELEASE);
        for (int q = 0; q < n_proj; q++)
            for (int w = 0; w < active; w++) __atomic_store_n(&sig[(size_t)q * n_workers + w], (int16_t)(base + stride * q + w), __ATOMIC_RELEASE);
        served_want += (long)n_proj * active;
        for (;;) {
            bool busy = false;
            for (auto &s : sig) busy = busy || __atomic_load_n(&s, __ATOMIC_ACQUIRE) != 0;
            if (!busy) break;
            std::this_thread::yield();
        }
        for (int q = 0; q < n_proj; q++)
            for (int b = 0; b < batch; b++)
                for (int t = 0; t < tkn; t++) {
                    std::vector<uint16_t> want((size_t)H);
                    const int a = slot_adapter[b];
                    scalar_lora(xs.data() + ((size_t)b * slot_tokens + t) * H, down[(size_t)q].data() + (size_t)a * H * r,
                                up[(size_t)q].data() + (size_t)a * r * H, nullptr, want.data(), H, H, r, 1.0f);
                    CHECK(memcmp(want.data(), outs[(size_t)q].data() + ((size_t)b * slot_tokens + t) * H, (size_t)H * 2) == 0,
                          "assist round %d projection %d request %d token %d differs", round, q, b, t);
                }
    }
    // a code that belongs to another cell, and one whose request lies beyond the slots: cleared, not served
    __atomic_store_n(&tkn_len, 16, __ATOMIC_RELEASE);                 // cpr = 4 -> worker 5 would serve request 1; fine.  Use a foreign code:
    __atomic_store_n(&sig[0], (int16_t)(base + 3), __ATOMIC_RELEASE);   // cell (0, 0) given row 3's code
    __atomic_store_n(&tkn_len, 1, __ATOMIC_RELEASE);                  // cpr = 1 -> worker 5 = request 5 >= n_slots
    __atomic_store_n(&sig[5], (int16_t)(base + 5), __ATOMIC_RELEASE);
    for (;;) {
        if (__atomic_load_n(&sig[0], __ATOMIC_ACQUIRE) == 0 && __atomic_load_n(&sig[5], __ATOMIC_ACQUIRE) == 0) break;
        std::this_thread::yield();
    }
    int64_t served = -1, rejected = -1;
    CHECK(mlora_cpu_assist_stop(srv, &served, &rejected) == 0, "assist stop");
    CHECK(served == served_want, "served %lld, expected %ld", (long long)served, served_want);
    CHECK(rejected == 2, "rejected %lld, expected 2", (long long)rejected);
    CHECK(outs[0][(size_t)3 * slot_tokens * H] == 0xdead, "a slot beyond the batch was written");
    mlora_cpu_pool_destroy(pool);
}

int main()
{
    test_pool();
    test_lora(37, 72, 56, 16, 3, 4, 8, true, 2.0f, 1);
    test_lora(9, 64, 64, 8, 2, 2, 3, false, 1.0f, 2);
    test_lora(21, 100, 44, 5, 4, 3, 4, true, 1.0f, 3);      // rank and width tails
    test_lora(13, 48, 80, 32, 2, 2, 64, false, 0.5f, 4);
    test_lora(6, 32, 24, 64, 1, 1, 2, true, 1.0f, 5);
    test_lora(5, 40, 40, 20, 2, 2, 2, false, 1.0f, 6);      // rank with no specialised path
    test_assist();
    if (g_failures) { fprintf(stderr, "%d check(s) failed\n", g_failures); return 1; }
    printf("selftest ok\n");
    return 0;
}
