// Measurement probe for bench.py, built into its own small library (libhqq_probe.so) and not part of the product
// ABI: a plain streaming read.  Every thread takes 128-bit words a grid stride apart, four in flight.  It computes
// nothing (the words are folded into one value that is stored only if it has an impossible bit pattern), so its
// duration is what the memory system needs to deliver `bytes` to a launch: the ceiling a GEMV over the same bytes
// is measured against.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512) void stream_read_kernel(const u32x4 *__restrict__ src, size_t n16, uint32_t *sink)
{
    u32x4 a = {0, 0, 0, 0};
    size_t i = (size_t)blockIdx.x * 512 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 512;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const u32x4 v0 = src[i], v1 = src[i + stride], v2 = src[i + 2 * stride], v3 = src[i + 3 * stride];
        a ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n16; i += stride)
        a ^= src[i];
    const uint32_t v = a.x ^ a.y ^ a.z ^ a.w;
    if (v == 0x9e3779b9u && (a.x & a.y & a.z) == 0x7f4a7c15u)
        sink[0] = v;
}

// src 16-byte aligned; sink_u32 one device word (never written in practice).  0 on success, -1 for a bad argument,
// else the HIP error of the launch.
extern "C" int hqq_probe_stream_read(const void *src, size_t bytes, void *sink_u32, void *stream)
{
    if (!src || !sink_u32 || (reinterpret_cast<uintptr_t>(src) & 15u))
        return -1;
    const size_t n16 = bytes / 16;
    if (n16 == 0)
        return 0;
    size_t blocks = (n16 + 4 * 512 - 1) / (4 * 512);
    blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    stream_read_kernel<<<dim3((unsigned)blocks), dim3(512), 0, (hipStream_t)stream>>>(static_cast<const u32x4 *>(src), n16,
                                                                                   static_cast<uint32_t *>(sink_u32));
    return static_cast<int>(hipGetLastError());
}
