/*
 * mlora_cpu.h -- C ABI of libmlora_cpu.so: the CPU side of the CPU-assisted LoRA path (host cores
 * compute the LoRA delta of a prefill batch while the adapter is still being loaded into the GPU pool).
 *
 * What each entry point replaces in the reference:
 *   - mlora_cpu_lora: the arithmetic of one CPU LoRA worker, `res = x.float() @ down @ up; out = res.half()`
 *     (lora_cpu/lora_shm_op/app.py:136-141), applied to every task of a batch; tasks are cut as the
 *     reference shards a request over workers, at most `tokens_per_task` tokens each
 *     (lightllm/models/lora_cpu.py:150-151: cpu_per_request = (tkn_num - 1) // cap + 1).
 *   - mlora_cpu_pool_create / destroy: the worker set.  The reference starts one pinned Python process per
 *     (request chunk, projection) (runServerCPULoRA.py:74-90) and keeps a mutex + condition-variable task
 *     queue in csrc/tpool.hpp:18-100; here one pool of persistent threads inside the serving process takes
 *     the tasks from one queue.
 *   - mlora_cpu_assist_start / stop: the polling loop of those workers (app.py:102-167) over the request
 *     slots, result slots and signal table of the transport (mlora_host_alloc / mlora_assist_export /
 *     mlora_assist_import in mlora.h), i.e. the worker side of csrc/async_lora.hpp:64-139.
 *
 * Plain host code: no GPU call anywhere in this library.  Pointers are host memory owned by the caller.
 * Return value: 0 or a negative MLORA_CPU_E* code; mlora_cpu_last_error() returns a thread-local message.
 *
 * Arithmetic contract: activations are IEEE binary16; weights are fp32 (the reference's, app.py:38-45) or
 * binary16; every product and sum is fp32, summed in ascending index order without fused multiply-add
 * (down projection over the Hin columns, up projection over the rank), one rounding to binary16 (nearest
 * even) at the end.  A token's result does not depend on how the batch is cut into tasks or on the number
 * of threads.
 */
#ifndef MLORA_CPU_H
#define MLORA_CPU_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLORA_CPU_OK 0
#define MLORA_CPU_EINVAL (-1)
#define MLORA_CPU_ERANGE (-2)
#define MLORA_CPU_ESTATE (-3)   /* pool or server handle not usable (NULL, stopped) */

#define MLORA_CPU_W_F32 0
#define MLORA_CPU_W_F16 1

#define MLORA_CPU_MAX_RANK 256
#define MLORA_CPU_MAX_THREADS 1024
#define MLORA_CPU_ASSIST_MAX_PROJ 4

const char *mlora_cpu_last_error(void);
int mlora_cpu_version(void);

/* Worker threads created once and woken per batch.  n_threads in 1..MLORA_CPU_MAX_THREADS; NULL on failure. */
void *mlora_cpu_pool_create(int n_threads);
void mlora_cpu_pool_destroy(void *pool);
int mlora_cpu_pool_threads(void *pool);

/*
 * LoRA delta on the host cores for T tokens:
 *     y[t] = half( (y0 ? float(y0[t]) : 0) + scale * (float(x[t]) . A_a) . B_a ),   a = tok_adapter[t]
 * x [T, Hin], y0 (may be NULL) and y [T, Hout] binary16; A [n_adapters, Hin, r] (the worker's `down`),
 * B [n_adapters, r, Hout] (`up`), fp32 or binary16 by w_dtype.  A token with a negative adapter id gets
 * y0 (or zeros); an id >= n_adapters is an error (MLORA_CPU_ERANGE, nothing written).
 * Tasks are runs of consecutive tokens with one adapter, cut to at most tokens_per_task tokens; they run on
 * `pool` (NULL: on the calling thread).  With scale == 1 and y0 == NULL this is the worker's expression.
 */
int mlora_cpu_lora(void *pool, const uint16_t *x, const void *A, const void *B, int w_dtype,
                   const int32_t *tok_adapter, const uint16_t *y0, uint16_t *y,
                   int T, int Hin, int Hout, int r, int n_adapters, float scale, int tokens_per_task);

/*
 * In-process workers of the CPU-assist transport.  A polling thread watches signals[q][w] (int16
 * [n_proj, n_workers]); a value v > 1 wakes worker w of projection q = (v - sig_base) / sig_stride with
 * row id v - sig_base - q * sig_stride, which serves request row / cpr, chunk row % cpr
 * (cpr = (tkn - 1) / cap + 1, tkn = tkn_len[0]): tokens [chunk * cap, min((chunk + 1) * cap, tkn)) of
 * x_slots [n_slots, slot_tokens, H] go through adapter slot_adapter[request] (NULL: adapter 0) of
 * down[q] [n_adapters, H, r] / up[q] [n_adapters, r, H] and land at the same rows of out_slots[q]; then the
 * signal is set to 0 (the reference's app.py:107-143 with the collector's placement, lora_cpu.py:210-232).
 * The chunk arithmetic runs on `pool`.  Codes that name a worker, request or token range outside the
 * buffers are counted as rejected and their signal is cleared without touching the slots.
 * mlora_cpu_assist_stop ends the polling thread after the chunks in flight; *served / *rejected (may be
 * NULL) receive the totals.  The buffers must stay valid between start and stop.
 */
void *mlora_cpu_assist_start(void *pool, const uint16_t *x_slots, uint16_t *const *out_slots,
                             int16_t *signals, const int32_t *tkn_len,
                             int n_proj, int n_workers, int n_slots, int slot_tokens, int H, int cap,
                             const void *const *down, const void *const *up, int w_dtype, int r, int n_adapters,
                             const int32_t *slot_adapter, int sig_base, int sig_stride);
int mlora_cpu_assist_stop(void *server, int64_t *served, int64_t *rejected);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_CPU_H */
