// CPU-assist transport for gfx950: the GPU side of the path on which host workers compute the LoRA
// delta while an adapter is still loading.  Three small kernels move 16-bit rows between device
// tensors and pinned host memory that is mapped into the device address space:
//   export : hidden states [B * tkn, H] -> request slots [n_slots, slot_tokens, H] on the host
//   signal : after the export, one wake-up code per worker into the host signal table
//   import : finished results [n_slots, slot_tokens, H] on the host -> [B, tkn, out] on the device,
//            the column slice [col0, col0 + out) of every row (the tensor-parallel rank's share)
// The kernels write and read host memory directly (16-byte accesses over the host link), so a
// whole batch takes one launch each way instead of one copy call per request and per chunk.
//
// Replaces Lora_CPU.invoke_lora_async (lightllm/models/lora_cpu.py:138-185: one cudaDtoHAsync per
// request, three cudaSignalDtoHAsync) and Lora_CPU.collect_qkv (lora_cpu.py:187-276: one
// cudaHtoD2D per finished chunk and projection) with the copy helpers of csrc/cuda_ops.hpp:109-229.
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

__global__ __launch_bounds__(256) void assist_export_kernel(const AssistArgs p)
{
    // one workgroup per (request, token); a row is H * 2 bytes
    const int b = blockIdx.x / p.tkn, t = blockIdx.x - b * p.tkn;
    const int chunks = p.H >> 3;
    const char *src = static_cast<const char *>(p.dev) + ((size_t)b * p.tkn + t) * p.H * 2;
    char *dst = static_cast<char *>(p.host_slots[0]) + ((size_t)b * p.slot_tokens + t) * p.H * 2;
    for (int c = threadIdx.x; c < chunks; c += 256) stg16(dst + (size_t)c * 16, ldg16_stream(src + (size_t)c * 16));
}

__global__ __launch_bounds__(256) void assist_signal_kernel(const AssistArgs p)
{
    // worker w of projection q is woken with the code sig_base + sig_stride * q + w (> 1)
    for (int e = threadIdx.x; e < p.n_proj * p.n_active; e += 256) {
        const int q = e / p.n_active, w = e - q * p.n_active;
        p.signals[(size_t)q * p.n_workers + w] = (int16_t)(p.sig_base + p.sig_stride * q + w);
    }
}

__global__ __launch_bounds__(256) void assist_import_kernel(const AssistArgs p)
{
    // one workgroup per (projection, request, token)
    const int per_proj = p.B * p.tkn;
    const int q = blockIdx.x / per_proj, rest = blockIdx.x - q * per_proj;
    const int b = rest / p.tkn, t = rest - b * p.tkn;
    const int chunks = p.out >> 3;
    const char *src = static_cast<const char *>(p.host_slots[q]) + (((size_t)b * p.slot_tokens + t) * p.H + p.col0) * 2;
    char *dst = static_cast<char *>(p.dev_out[q]) + ((size_t)b * p.tkn + t) * p.out * 2;
    for (int c = threadIdx.x; c < chunks; c += 256) stg16_stream(dst + (size_t)c * 16, ldg16(src + (size_t)c * 16));
}

int launch_assist_export(const AssistArgs &a, hipStream_t s)
{
    const long long rows = (long long)a.B * a.tkn;
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(assist_export_kernel, dim3((unsigned)rows), dim3(256), 0, s, a);
    int rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL(assist_signal_kernel, dim3(1), dim3(256), 0, s, a);
    return (int)hipGetLastError();
}

int launch_assist_import(const AssistArgs &a, hipStream_t s)
{
    const long long rows = (long long)a.n_proj * a.B * a.tkn;
    if (rows <= 0) return 0;
    hipLaunchKernelGGL(assist_import_kernel, dim3((unsigned)rows), dim3(256), 0, s, a);
    return (int)hipGetLastError();
}

}  // namespace mlora
