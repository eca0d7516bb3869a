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

// The same stream with a ring of four 16-byte loads per lane through a buffer resource: the loop has no branch (a
// request past the end of the workgroup's range returns zeros without touching memory), so its waits stay exact.
// 256 workgroups of this form reach a few percent more than the batched form above on the decoder's launch sizes;
// the harness takes the better of the two.
__global__ __launch_bounds__(kThreads) void hbm_stream_probe_ring_kernel(const u32x4 *__restrict__ p, size_t n16,
                                                                          u32x4 *__restrict__ sink)
{
#if defined(__HIP_DEVICE_COMPILE__)
    __shared__ u32x4 red[kThreads];
    const int tid = threadIdx.x;
    const size_t tiles = n16 / kThreads;                       // 8 KiB units
    const size_t mine = tiles / gridDim.x + (blockIdx.x < tiles % gridDim.x ? 1 : 0);
    const size_t first = (tiles / gridDim.x) * blockIdx.x + (blockIdx.x < tiles % gridDim.x ? blockIdx.x : tiles % gridDim.x);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4 *>(p) + first * kThreads, 0,
                                                                        (unsigned)(mine * kThreads * 16), 0x00020000);
    auto ld = [&](int tile) {
        return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, tid * 16, tile * (kThreads * 16), 2));
    };
    u32x4 r[4], acc = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 4; ++s)
        r[s] = ld(s);
    for (int t = 4; t < (int)mine + 4; t += 4) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            acc ^= r[s];
            r[s] = ld(t + s);
        }
    }
    red[tid] = acc;
    __syncthreads();
    if (tid < 64) {
        u32x4 s = red[tid];
        for (int w = 1; w < kThreads / 64; ++w)
            s ^= red[w * 64 + tid];
        sink[(size_t)blockIdx.x * 64 + tid] = s;
    }
#endif
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

// The ring form (see the kernel); a workgroup's range must stay under 4 GiB.
extern "C" int eet_hbm_stream_probe_ring(const void *src, size_t bytes, int workgroups, void *sink, size_t sink_bytes,
                                         void *stream)
{
    if (!src || !sink || workgroups <= 0 || workgroups > 65536 || reinterpret_cast<uintptr_t>(src) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(sink) % 16 != 0 || sink_bytes < (size_t)workgroups * 1024 ||
        bytes / (size_t)workgroups >= (1ull << 31))
        return -1;
    hipLaunchKernelGGL(hbm_stream_probe_ring_kernel, dim3(workgroups), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4 *>(src), bytes / 16, static_cast<u32x4 *>(sink));
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
