// The small kernels that sit between the GEMMs and the attention in a decoder
// layer: RMSnorm, fused-QKV split (+ NeoX rotary) that writes K and V straight
// into the KV cache, SwiGLU and the residual add.  All are launch-latency
// bound at decode sizes; they use 128-bit accesses and fp32 inner math.
#include <hip/hip_runtime.h>

#include <cmath>

#include "common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------------------
// RMSnorm: out = x * rsqrt(mean(x^2) + eps) * gamma.
// Replaces T5norm1_kernel_opt<half> (csrc/core/layer_norm.cu:490-531).
// One workgroup per row; each thread keeps its 8-element slices in registers.
// ---------------------------------------------------------------------------
constexpr int kNormThreads = 256;
constexpr int kNormMaxVec = 8;  // N <= 256 * 8 * 8 = 16384, the reference's limit (layer_norm.cu:588)

__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(const _Float16 *__restrict__ x,
                                                               const _Float16 *__restrict__ gamma,
                                                               _Float16 *__restrict__ out, int N, float eps)
{
    __shared__ float red[kNormThreads / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int nvec = N / 8;
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + (size_t)row * N);
    half8 v[kNormMaxVec];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            v[i] = __builtin_bit_cast(half8, xr[c]);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float f = (float)v[i][e];
                ss += f * f;
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        ss += __shfl_xor(ss, off, 64);
    if ((tid & 63) == 0)
        red[tid >> 6] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < kNormThreads / 64; ++w)
        tot += red[w];
    const float inv = rsqrtf(tot / (float)N + eps);
    const uint4 *gr = reinterpret_cast<const uint4 *>(gamma);
    uint4 *orow = reinterpret_cast<uint4 *>(out + (size_t)row * N);
#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            half8 g = __builtin_bit_cast(half8, gr[c]);
            half8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e)
                o[e] = (_Float16)((float)v[i][e] * inv * (float)g[e]);
            orow[c] = __builtin_bit_cast(uint4, o);
        }
    }
}

// ---------------------------------------------------------------------------
// The bias / LayerNorm branch of the ops.  One kernel: y = x [+ residual] [+ bias] with the
// reference's fp16 adds, then LayerNorm (gamma, beta: fp32 mean, then fp32 variance of the
// centred values, (y - mean) * rsqrt(var + eps) * gamma + beta, one rounding) or, with beta
// == nullptr, RMSnorm.  Covers decoder_norm1_kernel_opt<half> (csrc/core/layer_norm.cu:
// 384-446), add_bias_input_layernorm<half> (:39-80) and add_input_RMSnorm<half> (:103-131).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kNormThreads) void add_norm_kernel(const _Float16 *x,   // may be `out` (in place)
                                                                const _Float16 *__restrict__ residual,
                                                                const _Float16 *__restrict__ bias,
                                                                const _Float16 *__restrict__ gamma,
                                                                const _Float16 *__restrict__ beta,
                                                                _Float16 *out, int N, float eps)
{
    __shared__ float red[2][kNormThreads / 64];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int nvec = N / 8;
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + (size_t)row * N);
    const uint4 *rr = residual ? reinterpret_cast<const uint4 *>(residual + (size_t)row * N) : nullptr;
    const uint4 *br = reinterpret_cast<const uint4 *>(bias);
    half8 v[kNormMaxVec];
    float sum = 0.f, ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            v[i] = __builtin_bit_cast(half8, xr[c]);
            if (rr)
                v[i] = v[i] + __builtin_bit_cast(half8, rr[c]);   // fp16 add, then
            if (br)
                v[i] = v[i] + __builtin_bit_cast(half8, br[c]);   // a second fp16 add (:58)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)v[i][e];
                sum += f;
                ss += f * f;
            }
        }
    }
    auto block_sum = [&](float a, int slot) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
            a += __shfl_xor(a, off, 64);
        if ((tid & 63) == 0)
            red[slot][tid >> 6] = a;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < kNormThreads / 64; ++w)
            tot += red[slot][w];
        return tot;
    };
    float mean = 0.f, inv;
    if (beta != nullptr) {
        mean = block_sum(sum, 0) / (float)N;
        float var = 0.f;
#pragma unroll
        for (int i = 0; i < kNormMaxVec; ++i) {
            const int c = tid + i * kNormThreads;
            if (c < nvec) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float d = (float)v[i][e] - mean;
                    var += d * d;
                }
            }
        }
        inv = rsqrtf(block_sum(var, 1) / (float)N + eps);
    } else {
        inv = rsqrtf(block_sum(ss, 0) / (float)N + eps);
    }
    const uint4 *gr = reinterpret_cast<const uint4 *>(gamma);
    const uint4 *ber = reinterpret_cast<const uint4 *>(beta);
    uint4 *orow = reinterpret_cast<uint4 *>(out + (size_t)row * N);
#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            const half8 g = __builtin_bit_cast(half8, gr[c]);
            half8 o;
            if (beta != nullptr) {
                const half8 be = __builtin_bit_cast(half8, ber[c]);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    o[e] = (_Float16)(((float)v[i][e] - mean) * inv * (float)g[e] + (float)be[e]);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    o[e] = (_Float16)((float)v[i][e] * inv * (float)g[e]);
            }
            orow[c] = __builtin_bit_cast(uint4, o);
        }
    }
}

// out[m][:] += bias[:] in fp16 (add_bias, csrc/core/add_bias.cu:5-11)
__global__ void add_bias_kernel(_Float16 *__restrict__ out, const _Float16 *__restrict__ bias, size_t nvec, int nvec_row)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec)
        return;
    uint4 *o = reinterpret_cast<uint4 *>(out);
    const half8 b = __builtin_bit_cast(half8, reinterpret_cast<const uint4 *>(bias)[i % nvec_row]);
    o[i] = __builtin_bit_cast(uint4, __builtin_bit_cast(half8, o[i]) + b);
}

// ---------------------------------------------------------------------------
// Fused-QKV split.  qkv[B][S][3][H][dh] -> q_out[B][H][S][dh] and cache rows
// k_cache / v_cache[b][h][t0 + s][:].  With rope, pairs (i, i + dh/2) of q and
// k are rotated by angle pos / 10000^(2i/dh) in fp32 (csrc/core/common.cuh:
// 176-180, 209-225; kernel csrc/core/self_add_bias.cu:369-403), pos = s for
// the prompt and time_step for a decode step (:393).
// One thread handles 4 adjacent pairs, i.e. two 8-byte pieces of each of q,k,v.
// ---------------------------------------------------------------------------
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
constexpr int kRopeMaxPairs = 128;  // head sizes up to 256 keep their angles in LDS

__global__ void qkv_split_kernel(const _Float16 *__restrict__ qkv, _Float16 *__restrict__ q_out,
                                 _Float16 *__restrict__ k_cache, _Float16 *__restrict__ v_cache, int S, int H,
                                 int dh, int rope, int time_step, int t0, int T_cap)
{
    const int s = blockIdx.x, b = blockIdx.y;
    const int half_dh = dh / 2;
    const int per_head = half_dh / 4;  // threads per head
    // All heads of a row turn by the same dh/2 angles: computed once per workgroup.
    __shared__ float rot_cos[kRopeMaxPairs], rot_sin[kRopeMaxPairs];
    const bool table = rope && half_dh <= kRopeMaxPairs;
    if (table) {
        const float pos = (float)(time_step >= 0 ? time_step : s);
        for (int i = threadIdx.x; i < half_dh; i += blockDim.x) {
            const float ang = pos / powf(10000.0f, (float)(2 * i) / (float)dh);
            rot_cos[i] = cosf(ang);
            rot_sin[i] = sinf(ang);
        }
        __syncthreads();
    }
    for (int idx = threadIdx.x; idx < H * per_head; idx += blockDim.x) {
        const int h = idx / per_head, i0 = (idx % per_head) * 4;
        const size_t src = ((size_t)(b * S + s) * 3) * H * dh + (size_t)h * dh + i0;
        half4 q1 = *reinterpret_cast<const half4 *>(qkv + src);
        half4 q2 = *reinterpret_cast<const half4 *>(qkv + src + half_dh);
        half4 k1 = *reinterpret_cast<const half4 *>(qkv + src + (size_t)H * dh);
        half4 k2 = *reinterpret_cast<const half4 *>(qkv + src + (size_t)H * dh + half_dh);
        half4 v1 = *reinterpret_cast<const half4 *>(qkv + src + 2 * (size_t)H * dh);
        half4 v2 = *reinterpret_cast<const half4 *>(qkv + src + 2 * (size_t)H * dh + half_dh);
        if (rope) {
            const float pos = (float)(time_step >= 0 ? time_step : s);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float c, sn;
                if (table) {
                    c = rot_cos[i0 + e];
                    sn = rot_sin[i0 + e];
                } else {
                    const float ang = pos / powf(10000.0f, (float)(2 * (i0 + e)) / (float)dh);
                    c = cosf(ang);
                    sn = sinf(ang);
                }
                const float a = (float)q1[e], bq = (float)q2[e];
                q1[e] = (_Float16)(a * c - bq * sn);
                q2[e] = (_Float16)(bq * c + a * sn);
                const float ka = (float)k1[e], kb = (float)k2[e];
                k1[e] = (_Float16)(ka * c - kb * sn);
                k2[e] = (_Float16)(kb * c + ka * sn);
            }
        }
        const size_t qdst = (((size_t)b * H + h) * S + s) * dh + i0;
        *reinterpret_cast<half4 *>(q_out + qdst) = q1;
        *reinterpret_cast<half4 *>(q_out + qdst + half_dh) = q2;
        const size_t cdst = (((size_t)b * H + h) * T_cap + (t0 + s)) * dh + i0;
        *reinterpret_cast<half4 *>(k_cache + cdst) = k1;
        *reinterpret_cast<half4 *>(k_cache + cdst + half_dh) = k2;
        *reinterpret_cast<half4 *>(v_cache + cdst) = v1;
        *reinterpret_cast<half4 *>(v_cache + cdst + half_dh) = v2;
    }
}

// ---------------------------------------------------------------------------
// SwiGLU: gate <- up * gate / (1 + exp(-gate)).  Replaces gated_silu<half>
// (csrc/core/activation_kernel.cu:106-124); computed once in fp32 instead of
// the reference's half2 multiply and divide.
// ---------------------------------------------------------------------------
__global__ void swiglu_kernel(_Float16 *__restrict__ gate, const _Float16 *__restrict__ up, size_t nvec)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec)
        return;
    half8 g = __builtin_bit_cast(half8, reinterpret_cast<const uint4 *>(gate)[i]);
    half8 u = __builtin_bit_cast(half8, reinterpret_cast<const uint4 *>(up)[i]);
    half8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float x = (float)g[e];
        o[e] = (_Float16)((float)u[e] * x / (1.0f + expf(-x)));
    }
    reinterpret_cast<uint4 *>(gate)[i] = __builtin_bit_cast(uint4, o);
}

// out += residual (fp16 add).  Replaces add_input (csrc/core/add_bias.cu:22-28).
__global__ void residual_add_kernel(_Float16 *__restrict__ out, const _Float16 *__restrict__ res, size_t nvec)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec)
        return;
    half8 a = __builtin_bit_cast(half8, reinterpret_cast<const uint4 *>(out)[i]);
    half8 b = __builtin_bit_cast(half8, reinterpret_cast<const uint4 *>(res)[i]);
    reinterpret_cast<uint4 *>(out)[i] = __builtin_bit_cast(uint4, a + b);
}

// Beam-search cache reorder: dst[b] = src[index[b]] for the first `rows` time
// steps of every head, K and V in one launch.  Replaces reorderKV
// (csrc/core/transpose.cu:135-162), which gathers in place and says itself that
// the read / write order is not guaranteed; here source and destination are
// separate buffers, so the gather is exact for any index (duplicates included).
// An index outside [0, B) copies the beam's own rows.
// grid = (chunks, H, B); one (b, h) slab of rows*dh halves is contiguous.
__global__ __launch_bounds__(256) void kv_reorder_kernel(const _Float16 *__restrict__ k_src,
                                                         const _Float16 *__restrict__ v_src,
                                                         _Float16 *__restrict__ k_dst, _Float16 *__restrict__ v_dst,
                                                         const long long *__restrict__ index, int B, int H,
                                                         size_t slab_stride_vec, int nvec)
{
    const int b = blockIdx.z, h = blockIdx.y;
    long long from = index[b];
    if (from < 0 || from >= B)
        from = b;
    const size_t so = ((size_t)from * H + h) * slab_stride_vec, dst_o = ((size_t)b * H + h) * slab_stride_vec;
    const uint4 *ks = reinterpret_cast<const uint4 *>(k_src) + so, *vs = reinterpret_cast<const uint4 *>(v_src) + so;
    uint4 *kd = reinterpret_cast<uint4 *>(k_dst) + dst_o, *vd = reinterpret_cast<uint4 *>(v_dst) + dst_o;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < nvec; i += gridDim.x * 256) {
        const uint4 a = ks[i], c = vs[i];
        kd[i] = a;
        vd[i] = c;
    }
}

}  // namespace

extern "C" int eet_rmsnorm(const void *x, const void *gamma, void *out, int M, int N, float eps, void *stream)
{
    EET_REQUIRE(x && gamma && out, EET_ERR_INVALID_ARGUMENT, "eet_rmsnorm: null pointer");
    EET_REQUIRE(M >= 0 && N > 0, EET_ERR_INVALID_ARGUMENT, "eet_rmsnorm: bad sizes M=%d N=%d", M, N);
    EET_REQUIRE(N % 8 == 0 && N <= kNormThreads * kNormMaxVec * 8, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_rmsnorm: need N %% 8 == 0 and N <= 16384, got %d", N);
    if (M == 0)
        return EET_OK;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(M), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const _Float16 *>(x), static_cast<const _Float16 *>(gamma),
                       static_cast<_Float16 *>(out), N, eps);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_layernorm(const void *x, const void *gamma, const void *beta, void *out, int M, int N, float eps,
                             void *stream)
{
    EET_REQUIRE(x && gamma && beta && out, EET_ERR_INVALID_ARGUMENT, "eet_layernorm: null pointer");
    EET_REQUIRE(M >= 0 && N > 0, EET_ERR_INVALID_ARGUMENT, "eet_layernorm: bad sizes M=%d N=%d", M, N);
    EET_REQUIRE(N % 8 == 0 && N <= kNormThreads * kNormMaxVec * 8, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_layernorm: need N %% 8 == 0 and N <= 16384, got %d", N);
    if (M == 0)
        return EET_OK;
    hipLaunchKernelGGL(add_norm_kernel, dim3(M), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const _Float16 *>(x), static_cast<const _Float16 *>(nullptr),
                       static_cast<const _Float16 *>(nullptr), static_cast<const _Float16 *>(gamma),
                       static_cast<const _Float16 *>(beta), static_cast<_Float16 *>(out), N, eps);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_add_bias_residual_norm(void *out, const void *input, const void *bias, const void *gamma,
                                          const void *beta, int M, int N, float eps, void *stream)
{
    EET_REQUIRE(out && input && gamma, EET_ERR_INVALID_ARGUMENT, "eet_add_bias_residual_norm: null pointer");
    EET_REQUIRE(M >= 0 && N > 0, EET_ERR_INVALID_ARGUMENT, "eet_add_bias_residual_norm: bad sizes M=%d N=%d", M, N);
    EET_REQUIRE(N % 8 == 0 && N <= kNormThreads * kNormMaxVec * 8, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_add_bias_residual_norm: need N %% 8 == 0 and N <= 16384, got %d", N);
    if (M == 0)
        return EET_OK;
    hipLaunchKernelGGL(add_norm_kernel, dim3(M), dim3(kNormThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const _Float16 *>(out), static_cast<const _Float16 *>(input),
                       static_cast<const _Float16 *>(bias), static_cast<const _Float16 *>(gamma),
                       static_cast<const _Float16 *>(beta), static_cast<_Float16 *>(out), N, eps);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_add_bias(void *out, const void *bias, int M, int N, void *stream)
{
    EET_REQUIRE(out && bias, EET_ERR_INVALID_ARGUMENT, "eet_add_bias: null pointer");
    EET_REQUIRE(M >= 0 && N > 0, EET_ERR_INVALID_ARGUMENT, "eet_add_bias: bad sizes M=%d N=%d", M, N);
    EET_REQUIRE(N % 8 == 0, EET_ERR_UNSUPPORTED_SHAPE, "eet_add_bias: need N %% 8 == 0, got %d", N);
    const size_t nvec = (size_t)M * N / 8;
    if (nvec == 0)
        return EET_OK;
    hipLaunchKernelGGL(add_bias_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<_Float16 *>(out),
                       static_cast<const _Float16 *>(bias), nvec, N / 8);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_qkv_split(const void *qkv, void *q_out, void *k_cache, void *v_cache, int B, int S, int H, int dh,
                             int rope, int time_step, int t0, int T_cap, void *stream)
{
    EET_REQUIRE(qkv && q_out && k_cache && v_cache, EET_ERR_INVALID_ARGUMENT, "eet_qkv_split: null pointer");
    EET_REQUIRE(B >= 0 && S >= 0 && H > 0 && dh > 0 && t0 >= 0, EET_ERR_INVALID_ARGUMENT,
                "eet_qkv_split: bad sizes B=%d S=%d H=%d dh=%d t0=%d", B, S, H, dh, t0);
    EET_REQUIRE(dh % 8 == 0, EET_ERR_UNSUPPORTED_SHAPE, "eet_qkv_split: head size %d must be a multiple of 8", dh);
    EET_REQUIRE(t0 + S <= T_cap, EET_ERR_INVALID_ARGUMENT,
                "eet_qkv_split: rows [%d, %d) exceed the cache capacity %d", t0, t0 + S, T_cap);
    EET_REQUIRE(B <= 65535, EET_ERR_UNSUPPORTED_SHAPE, "eet_qkv_split: batch %d too large", B);
    if (B == 0 || S == 0)
        return EET_OK;
    const int work = H * (dh / 8);
    const int threads = work >= 256 ? 256 : ((work + 63) / 64) * 64;
    hipLaunchKernelGGL(qkv_split_kernel, dim3(S, B), dim3(threads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const _Float16 *>(qkv), static_cast<_Float16 *>(q_out),
                       static_cast<_Float16 *>(k_cache), static_cast<_Float16 *>(v_cache), S, H, dh, rope, time_step,
                       t0, T_cap);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

static int elementwise_args(const char *fn, const void *a, const void *b, int M, int N)
{
    EET_REQUIRE(a && b, EET_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    EET_REQUIRE(M >= 0 && N > 0, EET_ERR_INVALID_ARGUMENT, "%s: bad sizes M=%d N=%d", fn, M, N);
    EET_REQUIRE(N % 8 == 0, EET_ERR_UNSUPPORTED_SHAPE, "%s: need N %% 8 == 0, got %d", fn, N);
    return EET_OK;
}

extern "C" int eet_swiglu(void *gate, const void *up, int M, int N, void *stream)
{
    if (int rc = elementwise_args("eet_swiglu", gate, up, M, N))
        return rc;
    const size_t nvec = (size_t)M * N / 8;
    if (nvec == 0)
        return EET_OK;
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<_Float16 *>(gate),
                       static_cast<const _Float16 *>(up), nvec);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_residual_add(void *out, const void *residual, int M, int N, void *stream)
{
    if (int rc = elementwise_args("eet_residual_add", out, residual, M, N))
        return rc;
    const size_t nvec = (size_t)M * N / 8;
    if (nvec == 0)
        return EET_OK;
    hipLaunchKernelGGL(residual_add_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<_Float16 *>(out),
                       static_cast<const _Float16 *>(residual), nvec);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" int eet_kv_cache_reorder(const void *k_src, const void *v_src, void *k_dst, void *v_dst,
                                    const int64_t *reorder_index, int B, int H, int dh, int rows, int T_cap,
                                    void *stream)
{
    EET_REQUIRE(k_src && v_src && k_dst && v_dst && reorder_index, EET_ERR_INVALID_ARGUMENT,
                "eet_kv_cache_reorder: null pointer");
    EET_REQUIRE(B >= 0 && H > 0 && dh > 0 && rows >= 0 && rows <= T_cap, EET_ERR_INVALID_ARGUMENT,
                "eet_kv_cache_reorder: bad sizes B=%d H=%d dh=%d rows=%d T_cap=%d", B, H, dh, rows, T_cap);
    EET_REQUIRE(dh % 8 == 0, EET_ERR_UNSUPPORTED_SHAPE, "eet_kv_cache_reorder: head size %d must be a multiple of 8",
                dh);
    EET_REQUIRE(B <= 65535 && H <= 65535, EET_ERR_UNSUPPORTED_SHAPE, "eet_kv_cache_reorder: B=%d / H=%d too large", B,
                H);
    // The gather reads beams that other workgroups write: in place it would race.
    const size_t bytes = (size_t)B * H * T_cap * dh * sizeof(_Float16);
    auto overlap = [bytes](const void *a, const void *b) {
        const char *x = static_cast<const char *>(a), *y = static_cast<const char *>(b);
        return x < y + bytes && y < x + bytes;
    };
    EET_REQUIRE(!overlap(k_src, k_dst) && !overlap(v_src, v_dst) && !overlap(k_src, v_dst) && !overlap(v_src, k_dst),
                EET_ERR_INVALID_ARGUMENT, "eet_kv_cache_reorder: source and destination caches overlap");
    if (B == 0 || rows == 0)
        return EET_OK;
    const int nvec = rows * (dh / 8);
    int chunks = (nvec + 1023) / 1024;      // >= 4 vectors per thread, all beams and heads in flight
    if (chunks < 1)
        chunks = 1;
    hipLaunchKernelGGL(kv_reorder_kernel, dim3(chunks, H, B), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const _Float16 *>(k_src), static_cast<const _Float16 *>(v_src),
                       static_cast<_Float16 *>(k_dst), static_cast<_Float16 *>(v_dst),
                       reinterpret_cast<const long long *>(reorder_index), B, H, (size_t)T_cap * (dh / 8), nvec);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}
