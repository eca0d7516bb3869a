// The offline packer on the GPU: fp16 / fp32 [K][N] weights already resident in
// HBM -> per-output-channel int8 + scales -> gfx950 tile layout, in two passes.
//
// Same results, bit for bit, as eet_quantize_int8 followed by eet_pack_gfx950
// (packer.cc), i.e. as the reference's symmetric_quantize
// (3rdparty/cutlass_kernels/cutlass_preprocessors.cc:581-678) in
// EET_QUANT_REF128 mode: every step is a single correctly rounded IEEE fp32
// operation (|x| and max, one multiply or divide for the scale, one divide per
// weight, an exact round-half-away), so host and device cannot differ.  The
// reference has no device quantiser; converting a checkpoint on the host costs
// seconds per billion weights, here the time of reading it twice from HBM.
//
// HBM-bound.  Pass 1 reads the matrix once (column absmax, one 32-bit atomic
// max per column and 128-row chunk); pass 2 reads it again (from the Infinity
// Cache when it fits) and writes one byte per weight in the packed layout, plus
// one more in row-major order when the caller wants the unprocessed matrix.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kColsPerThread = 8;   // pass 1: 16 bytes of fp16 per load
constexpr int kMaxRows = 128;       // rows per workgroup in pass 1 (32 per wavefront)
constexpr int kTileCols = 128;      // pass 2: one k-tile x 8 n-tiles per workgroup

template <typename T>
__device__ __forceinline__ float to_f32(T x)
{
    return static_cast<float>(x);
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t *p, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n)
        p[i] = 0u;
}

// amax[c] = max over rows of |w[r][c]|, as the bit pattern of a non-negative
// float (which orders like the unsigned integer).  NaN weights are ignored, as
// on the host (the comparison is false).  The four wavefronts of a workgroup
// share 512 columns and take every fourth row, eight loads in flight each; they
// meet in LDS, so one atomic per column leaves the workgroup.
template <typename T>
__global__ __launch_bounds__(256) void colmax_kernel(const T *__restrict__ w, size_t K, size_t N,
                                                     uint32_t *__restrict__ amax)
{
    __shared__ float part[4][64 * kColsPerThread];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t c0 = ((size_t)blockIdx.x * 64 + lane) * kColsPerThread;
    const size_t r0 = (size_t)blockIdx.y * kMaxRows;
    const size_t r1 = r0 + kMaxRows < K ? r0 + kMaxRows : K;
    float m[kColsPerThread];
#pragma unroll
    for (int i = 0; i < kColsPerThread; ++i)
        m[i] = 0.f;
    if (c0 < N) {   // N % 16 == 0: the 8 columns are in range together
        for (size_t r = r0 + wave; r < r1; r += 32) {
            T v[8][kColsPerThread];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const size_t rr = r + 4 * u < r1 ? r + 4 * u : r;   // past the end: the row again
                __builtin_memcpy(v[u], w + rr * N + c0, sizeof(v[u]));
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int i = 0; i < kColsPerThread; ++i) {
                    const float a = __builtin_fabsf(to_f32(v[u][i]));
                    m[i] = (m[i] < a) ? a : m[i];
                }
        }
    }
#pragma unroll
    for (int i = 0; i < kColsPerThread; ++i)
        part[wave][lane * kColsPerThread + i] = m[i];
    __syncthreads();
    for (int c = threadIdx.x; c < 64 * kColsPerThread; c += 256) {
        const size_t col = (size_t)blockIdx.x * 64 * kColsPerThread + c;
        if (col < N) {
            float a = part[0][c];
            a = a < part[1][c] ? part[1][c] : a;
            a = a < part[2][c] ? part[2][c] : a;
            a = a < part[3][c] ? part[3][c] : a;
            atomicMax(amax + col, __float_as_uint(a));
        }
    }
}

// round-half-away-from-zero of x / s clamped to [lo, 127]; see quant_row in
// packer.cc for why this equals clamp(round(x / s)).
__device__ __forceinline__ int quant_one(float x, float s, float nan_to, int lo)
{
    float v = __fdiv_rn(x, s);
    v = (v == v) ? v : nan_to;
    v = (v < 200.f) ? v : 200.f;
    v = (v > -200.f) ? v : -200.f;
    int t = static_cast<int>(v);
    const float d = v - static_cast<float>(t);
    t += (d >= 0.5f) ? 1 : 0;
    t -= (d <= -0.5f) ? 1 : 0;
    t = (t < 127) ? t : 127;
    t = (t > lo) ? t : lo;
    return t;
}

// The same value without a division per weight (the kernel would be bound by
// the vector ALU otherwise): r = x * (1 / s) is within 2^-23 relative, i.e.
// 1.5e-5 absolute for |r| <= 128, of the exact quotient, and so is the
// correctly rounded x / s.  Unless the fractional part of |r| lies within 1e-4
// of 0.5 both therefore round to the same integer, and adding 0.5 in fp32
// cannot carry r across an integer either.  The rare weights near a tie, and
// anything not finite (0 / 0 in an all-zero column), take the exact path.
__device__ __forceinline__ int quant_fast(float x, float s, float inv_s, float nan_to, int lo)
{
    const float r = x * inv_s;
    const float a = __builtin_fabsf(r);
    const float f = a - __builtin_floorf(a);
    if (!(__builtin_fabsf(f - 0.5f) > 1e-4f) || !(a < 130.f))
        return quant_one(x, s, nan_to, lo);
    int t = static_cast<int>(r + __builtin_copysignf(0.5f, r));
    t = (t < 127) ? t : 127;
    t = (t > lo) ? t : lo;
    return t;
}

// One k-tile (64 rows) x 128 columns per workgroup: rows are read in 256-byte
// (fp16) pieces and quantised; the tile is kept column-major in LDS (a thread
// owns 4 consecutive rows of its 8 columns, i.e. 8 whole 32-bit words), so that
// the 16 bytes lane (g, i) of a packed tile holds -- q[64*kt + 16*g + b][16*nt
// + i] ^ 0x80 for b = 0 .. 15, the layout of eet_pack_gfx950 -- are four
// consecutive words, and the tile leaves as eight whole 1 KiB packed tiles.
template <typename T>
__global__ __launch_bounds__(256) void quant_pack_kernel(const T *__restrict__ w, size_t K, size_t N, int ref128,
                                                         const uint32_t *__restrict__ amax, int8_t *__restrict__ q_out,
                                                         uint8_t *__restrict__ packed, T *__restrict__ scale)
{
    __shared__ uint32_t lq[kTileCols][17];   // [column][4-row word], one word of padding per column
    const size_t kt = blockIdx.y, ktiles = K / 64;
    const size_t col0 = (size_t)blockIdx.x * kTileCols;
    const int tid = threadIdx.x;
    const int c8 = (tid & 15) * 8, rw = tid >> 4;   // columns c8 .. c8+7, rows 4*rw .. 4*rw+3
    const size_t col = col0 + c8;
    const float nan_to = ref128 ? 1000.f : 0.f;
    const int lo = ref128 ? -128 : -127;

    if (col < N) {   // N % 16 == 0: the 8 columns are in range together
        float s[8], inv_s[8];
        uint32_t am[8];
        __builtin_memcpy(am, amax + col, sizeof(am));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float a = __uint_as_float(am[i]);
            s[i] = ref128 ? a * (1.f / 128.f) : __fdiv_rn(a, 127.f);
            inv_s[i] = __fdiv_rn(1.f, s[i]);
        }
        if (kt == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                scale[col + i] = static_cast<T>(s[i]);
        }
        T v[4][8];
#pragma unroll
        for (int it = 0; it < 4; ++it)
            __builtin_memcpy(v[it], w + (kt * 64 + 4 * rw + it) * N + col, sizeof(v[it]));
        uint32_t word[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            union {
                int8_t b[8];
                u32x2 u;
            } o;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int t = quant_fast(to_f32(v[it][i]), s[i], inv_s[i], nan_to, lo);
                o.b[i] = static_cast<int8_t>(t);
                word[i] |= (static_cast<uint32_t>(t) & 0xffu) << (8 * it);
            }
            if (q_out != nullptr)
                *reinterpret_cast<u32x2 *>(q_out + (kt * 64 + 4 * rw + it) * N + col) = o.u;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
            lq[c8 + i][rw] = word[i] ^ 0x80808080u;
    }
    __syncthreads();
    // 8 tiles x 64 lanes = 512 pieces of 16 bytes, two per thread
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int piece = it * 256 + tid;
        const int n8 = piece >> 6, lane = piece & 63;
        const int g = lane >> 4, i = lane & 15;
        const size_t nt = col0 / 16 + n8;
        if (nt * 16 >= N)
            continue;
        const uint32_t *src = &lq[n8 * 16 + i][4 * g];
        const u32x4 o = {src[0], src[1], src[2], src[3]};
        *reinterpret_cast<u32x4 *>(packed + (nt * ktiles + kt) * 1024 + lane * 16) = o;
    }
}

template <typename T>
int run(const void *w, size_t K, size_t N, int mode, int8_t *q, int8_t *packed, void *scale, uint32_t *amax,
        hipStream_t st)
{
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, st, amax, N);
    EET_HIP_CHECK(hipGetLastError());
    const dim3 g1((unsigned)((N + 64 * kColsPerThread - 1) / (64 * kColsPerThread)),
                  (unsigned)((K + kMaxRows - 1) / kMaxRows));
    hipLaunchKernelGGL(colmax_kernel<T>, g1, dim3(256), 0, st, static_cast<const T *>(w), K, N, amax);
    EET_HIP_CHECK(hipGetLastError());
    const dim3 g2((unsigned)((N + kTileCols - 1) / kTileCols), (unsigned)(K / 64));
    hipLaunchKernelGGL(quant_pack_kernel<T>, g2, dim3(256), 0, st, static_cast<const T *>(w), K, N,
                       mode == EET_QUANT_REF128 ? 1 : 0, amax, q, reinterpret_cast<uint8_t *>(packed),
                       static_cast<T *>(scale));
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

}  // namespace

extern "C" size_t eet_quantize_pack_device_workspace(size_t N) { return N * sizeof(uint32_t); }

extern "C" int eet_quantize_pack_device(const void *w, int w_dtype, size_t K, size_t N, int mode, int8_t *q,
                                        int8_t *packed, void *scale, void *workspace, size_t workspace_bytes,
                                        void *stream)
{
    EET_REQUIRE(w && packed && scale, EET_ERR_INVALID_ARGUMENT, "eet_quantize_pack_device: null pointer");
    EET_REQUIRE(w_dtype == EET_DTYPE_F32 || w_dtype == EET_DTYPE_F16, EET_ERR_INVALID_ARGUMENT,
                "eet_quantize_pack_device: w_dtype must be EET_DTYPE_F32 or EET_DTYPE_F16, got %d", w_dtype);
    EET_REQUIRE(mode == EET_QUANT_REF128 || mode == EET_QUANT_SYM127, EET_ERR_INVALID_ARGUMENT,
                "eet_quantize_pack_device: unknown mode %d", mode);
    EET_REQUIRE(K > 0 && N > 0 && K % 64 == 0 && N % 16 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_quantize_pack_device: need K %% 64 == 0 and N %% 16 == 0, got K=%zu N=%zu", K, N);
    EET_REQUIRE(K / 64 <= 65535 && (K + kMaxRows - 1) / kMaxRows <= 65535, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_quantize_pack_device: K = %zu exceeds the grid limit", K);
    EET_REQUIRE((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(packed)) % 16 == 0 &&
                    (q == nullptr || reinterpret_cast<uintptr_t>(q) % 8 == 0),
                EET_ERR_INVALID_ARGUMENT, "eet_quantize_pack_device: w and packed need 16-byte, q 8-byte alignment");
    EET_REQUIRE(workspace != nullptr && workspace_bytes >= N * sizeof(uint32_t) &&
                    reinterpret_cast<uintptr_t>(workspace) % 4 == 0,
                EET_ERR_WORKSPACE, "eet_quantize_pack_device: workspace of %zu bytes needed, %zu given",
                N * sizeof(uint32_t), workspace_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (w_dtype == EET_DTYPE_F32)
        return run<float>(w, K, N, mode, q, packed, scale, static_cast<uint32_t *>(workspace), st);
    return run<_Float16>(w, K, N, mode, q, packed, scale, static_cast<uint32_t *>(workspace), st);
}
