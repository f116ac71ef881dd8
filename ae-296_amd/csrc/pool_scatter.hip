// Adapter swap-in, device side: rank rows arrive from the host as one contiguous block per
// (layer, projection, side) and are placed on the pages the adapter owns in the pool slabs.
// One workgroup per (job, rank row): a row is copied with 16-byte nontemporal loads and stores.
// The page ids travel in the kernel arguments, so the copy does not depend on when the device
// copy of the page table is refreshed.
//
// Replaces the whole-tensor copies of the reference's swapper (shared_tensor.py:117-147, one
// host->device copy and one slice assignment per layer and tensor) and of load_lora_prefill
// (lightllm/models/lora_gpu.py:165-188).
#include "mlora_args.hpp"
#include "mlora_dev.hpp"

namespace mlora {

__global__ __launch_bounds__(256) void scatter_kernel(const ScatterArgs p)
{
    const int job = blockIdx.x / p.rank, j = blockIdx.x - job * p.rank;
    const int pg = p.pages[j >> p.page_shift];
    if (pg < 0 || pg >= p.n_pages) return;                      // checked on the host too
    const long long row = ((long long)pg << p.page_shift) + (j & ((1 << p.page_shift) - 1));
    const int chunks = p.row_bytes[job] >> 4;
    const char *src = static_cast<const char *>(p.src[job]) + (size_t)j * p.row_bytes[job];
    char *dst = static_cast<char *>(p.dst[job]) + (size_t)row * p.row_bytes[job];
    for (int c = threadIdx.x; c < chunks; c += 256) stg16_stream(dst + (size_t)c * 16, ldg16_stream(src + (size_t)c * 16));
}

int launch_scatter(const ScatterArgs &a, hipStream_t s)
{
    const long long total = (long long)a.n_jobs * a.rank;
    if (total <= 0) return 0;
    hipLaunchKernelGGL(scatter_kernel, dim3((unsigned)total), dim3(256), 0, s, a);
    return (int)hipGetLastError();
}

}  // namespace mlora
