// Measurement utility: a read-only streaming kernel with the launch structure of
// the small-M GEMM (contiguous range per workgroup, 128-bit non-temporal loads,
// two batches in flight, one LDS reduction and one small store at the end).
// bench.py launches it over the same weight buffers, in the same order and with
// the same grids as the GEMM pass: what it reaches is what this machine allows a
// chain of dependent launches of those sizes, i.e. the practical ceiling the
// GEMM's HBM rate is to be read against (next to the published 8 TB/s).
// No counterpart in the reference and no part of the operator interface.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kThreads = 512, kU = 4;

__global__ __launch_bounds__(kThreads) void hbm_stream_probe_kernel(const u32x4 *__restrict__ p, size_t n16,
                                                                     u32x4 *__restrict__ sink)
{
    __shared__ u32x4 red[kThreads];
    const int tid = threadIdx.x;
    // whole batches of kThreads * kU vectors, dealt round-robin to the workgroups
    const size_t batches = n16 / (kThreads * kU);
    const size_t mine = batches / gridDim.x + (blockIdx.x < batches % gridDim.x ? 1 : 0);
    const size_t first = (batches / gridDim.x) * blockIdx.x + (blockIdx.x < batches % gridDim.x ? blockIdx.x : batches % gridDim.x);
    const u32x4 *q = p + first * (kThreads * kU) + tid;
    u32x4 a[kU], b[kU], acc = {0, 0, 0, 0};
    auto req = [&](u32x4(&dst)[kU], size_t i) {
        if (i < mine) {
#pragma unroll
            for (int u = 0; u < kU; ++u)
                dst[u] = __builtin_nontemporal_load(q + i * (kThreads * kU) + u * kThreads);
        } else {
#pragma unroll
            for (int u = 0; u < kU; ++u)
                dst[u] = u32x4{0, 0, 0, 0};
        }
    };
    req(a, 0);
    req(b, 1);
    for (size_t i = 2; i < mine + 2; i += 2) {
#pragma unroll
        for (int u = 0; u < kU; ++u)
            acc ^= a[u];
        req(a, i);
#pragma unroll
        for (int u = 0; u < kU; ++u)
            acc ^= b[u];
        req(b, i + 1);
    }
    red[tid] = acc;
    __syncthreads();
    if (tid < 64) {
        u32x4 s = red[tid];
        for (int w = 1; w < kThreads / 64; ++w)
            s ^= red[w * 64 + tid];
        sink[(size_t)blockIdx.x * 64 + tid] = s;
    }
}

}  // namespace

// Built into libeet_bench.so, not into the product library: bench.py binds it directly.
// Returns 0, or -1 for bad arguments, -3 for a failed launch.
extern "C" int eet_hbm_stream_probe(const void *src, size_t bytes, int workgroups, void *sink, size_t sink_bytes,
                                    void *stream)
{
    if (!src || !sink || workgroups <= 0 || workgroups > 65536 || reinterpret_cast<uintptr_t>(src) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(sink) % 16 != 0 || sink_bytes < (size_t)workgroups * 1024)
        return -1;   // sink: 1 KiB of device memory per workgroup
    hipLaunchKernelGGL(hbm_stream_probe_kernel, dim3(workgroups), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4 *>(src), bytes / 16, static_cast<u32x4 *>(sink));
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
