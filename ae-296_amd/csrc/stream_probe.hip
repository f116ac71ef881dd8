// Streaming probe: what a plain pass over device memory reaches on this device, measured by the benchmark in
// the same run as the LoRA kernels so that their figures can be read against the box's own ceiling (which
// differs from box to box and lies well under the published HBM peak).  MODE 0 reads every 16 bytes once with
// the nontemporal loads the LoRA kernels use; MODE 1 reads, changes and writes back in place (the access
// pattern of an accumulate-into-y expand); MODE 2 reads everything and writes back one 2 KiB piece in ten (the
// mix of a decode expand: B rows read once, a tenth as many bytes of y read and written).  No counterpart in the
// reference.  Built into its own small library
// (libmlora_probe.so) that only the benchmark loads: it is a measuring aid, not part of the operator surface.
#include "mlora_dev.hpp"

namespace mlora {

template <int MODE>
__global__ __launch_bounds__(256) void stream_probe_kernel(uint4 *__restrict__ p, long long n16, unsigned *__restrict__ sink)
{
    constexpr int U = 8;                                   // 16-byte loads in flight per thread
    const long long stride = (long long)gridDim.x * 256 * U;
    unsigned acc = 0;
    for (long long i = (long long)blockIdx.x * 256 * U + threadIdx.x; i < n16; i += stride) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const long long idx = i + (long long)u * 256;
            v[u] = idx < n16 ? ldg16_stream(p + idx) : zero16();
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const long long idx = i + (long long)u * 256;
            if constexpr (MODE == 0) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
            else if (MODE == 1 && idx < n16) { v[u].x += 1u; stg16_stream(p + idx, v[u]); }
            else if (MODE == 2) {
                if (idx < n16 && (idx >> 7) % 10 == 0) { v[u].x += 1u; stg16_stream(p + idx, v[u]); }
                else acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
            }
        }
    }
    if (MODE != 1 && acc == 0x9e3779b9u && sink) sink[0] = acc;      // keeps the loads alive; practically never taken
}

static int launch_stream_probe(void *p, long long bytes, int mode, unsigned *sink, hipStream_t s)
{
    const long long n16 = bytes / 16;
    if (n16 <= 0) return 0;
    long long blocks = (n16 + 256 * 8 - 1) / (256 * 8);
    if (blocks > 2048) blocks = 2048;                      // eight workgroups per compute unit, each striding over the buffer
    if (mode == 0) hipLaunchKernelGGL(stream_probe_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<uint4 *>(p), n16, sink);
    else if (mode == 1) hipLaunchKernelGGL(stream_probe_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<uint4 *>(p), n16, sink);
    else hipLaunchKernelGGL(stream_probe_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<uint4 *>(p), n16, sink);
    return (int)hipGetLastError();
}

}  // namespace mlora

// One plain streaming pass over `bytes` of device memory at `buf` (16-byte aligned) on `stream`: mode 0 reads every
// 16 bytes once, mode 1 adds 1 to the first 32-bit word of every 16 bytes in place, mode 2 does that for one 2 KiB
// piece in ten and only reads the others.  Returns 0, -1 for a bad
// argument, or the HIP error of the launch.
extern "C" int mlora_probe_stream(void *buf, long long bytes, int mode, void *stream)
{
    if (bytes < 0 || mode < 0 || mode > 2) return -1;
    if (bytes == 0) return 0;
    if (!buf || (reinterpret_cast<uintptr_t>(buf) & 15u)) return -1;
    return mlora::launch_stream_probe(buf, bytes, mode, nullptr, static_cast<hipStream_t>(stream));
}
