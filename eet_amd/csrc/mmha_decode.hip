// Masked multi-head decode attention over the fp16 KV cache (one new token per
// sequence), with an optional ALiBi bias row.
//
// Replaces masked_attention_kernel_opt (csrc/core/attention_dispatch.cu:140-324,
// dispatcher :888-928) and t5_masked_attention_kernel (:1155-1336, dispatcher
// :1397-1424).  Semantics kept: logit = (q . k_t) * half(1/sqrt(dh)) [+ bias],
// rows t < pad[b] carry no weight, softmax denominator + 1e-6, fp32 math.
// Not kept: the reference rounds each logit to fp16 (:238) and caps step at
// 4096 by a static shared array (:164).
//
// HBM-bound: K and V rows (dh halves, contiguous) are each read exactly once
// with 128-bit loads.  The cache is [B_cap][H][T_cap][dh], so one (b, h) pair
// streams one contiguous range.  The time axis is split over `nsplit`
// workgroups per (b, h) so that a few hundred heads still fill 256 CUs
// (the reference runs one block per head); every workgroup produces an
// un-normalised partial (max, sum, acc[dh]) and a second small kernel merges
// them.  With nsplit == 1 the first kernel writes the context itself.
// Inside a workgroup every group of dh/8 lanes streams its own rows with a
// running softmax, K and V rows requested together several rows deep; there
// is no per-launch limit on step.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdlib>

#include "common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;

__device__ __forceinline__ float dot8(const u32x4 &a, const u32x4 &b)
{
    const half8 ha = __builtin_bit_cast(half8, a), hb = __builtin_bit_cast(half8, b);
    float s = 0.f;
    s = __builtin_amdgcn_fdot2(__builtin_shufflevector(ha, ha, 0, 1), __builtin_shufflevector(hb, hb, 0, 1), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_shufflevector(ha, ha, 2, 3), __builtin_shufflevector(hb, hb, 2, 3), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_shufflevector(ha, ha, 4, 5), __builtin_shufflevector(hb, hb, 4, 5), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_shufflevector(ha, ha, 6, 7), __builtin_shufflevector(hb, hb, 6, 7), s, false);
    return s;
}

// Decode streams every cache row exactly once: non-temporal loads.
__device__ __forceinline__ u32x4 load_row16(const u32x4 *p)
{
    return __builtin_nontemporal_load(p);
}

template <int WIDTH>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = WIDTH / 2; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float block_reduce(float v, bool is_max, float *scratch)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float o = __shfl_xor(v, off, 64);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    if (lane == 0)
        scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w)
        r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    __syncthreads();
    return r;
}

// NeoX rotary on one 8-element slice.  x holds elements d = 8*sub .. 8*sub+7 of
// a head row, y the slice DH/2 away; rope_row is [cos(DH/2) | sin(DH/2)] for the
// position.  fp32 math, one rounding to fp16 (csrc/core/common.cuh:209-225).
template <int DH>
__device__ __forceinline__ u32x4 rotate8(const u32x4 &x, const u32x4 &y, int sub, const float *rope_row)
{
    constexpr int LPR = DH / 8;
    const bool lower = sub < LPR / 2;
    const int i0 = (sub % (LPR / 2)) * 8;
    const half8 hx = __builtin_bit_cast(half8, x), hy = __builtin_bit_cast(half8, y);
    half8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float c = rope_row[i0 + e], sn = rope_row[DH / 2 + i0 + e];
        const float a = (float)hx[e], b = (float)hy[e];
        o[e] = (_Float16)(lower ? a * c - b * sn : a * c + b * sn);
    }
    return __builtin_bit_cast(u32x4, o);
}

// DH: head size.  LPR = DH/8 lanes cover one row with one 16-byte load each.
// One query per (b, h) attends rows [0, step); grid = (B*H, nsplit).
template <int DH, int UN>
__global__ __launch_bounds__(kThreads) void mmha_decode_split_kernel(
    const _Float16 *__restrict__ q, const _Float16 *__restrict__ k_new, const _Float16 *__restrict__ v_new,
    long qkv_stride, _Float16 *__restrict__ k_cache, _Float16 *__restrict__ v_cache, _Float16 *__restrict__ ctx,
    const _Float16 *__restrict__ alibi, const int64_t *__restrict__ pad, float *__restrict__ partial, int H,
    int step, int T_cap, int nsplit, float scale, const float *__restrict__ rope_row)
{
    constexpr int LPR = DH / 8;            // lanes per row
    constexpr int RPB = kThreads / LPR;    // row streams of the block (one per group of LPR lanes)
    __shared__ float accs[RPB][DH + 1];
    __shared__ float stream_m[RPB], stream_l[RPB];

    const int split = blockIdx.y;
    const int bh = blockIdx.x;
    const int alibi_ld = step;
    const int b = bh / H, h = bh % H;
    const int tid = threadIdx.x;
    const int sub = tid % LPR;   // which 8-element slice of the row
    const int rs = tid / LPR;    // which row stream

    const size_t qoff = qkv_stride ? (size_t)b * qkv_stride + (size_t)h * DH : (size_t)bh * DH;
    const size_t coff = (size_t)bh * DH;
    _Float16 *kc = k_cache + ((size_t)b * H + h) * (size_t)T_cap * DH;
    _Float16 *vc = v_cache + ((size_t)b * H + h) * (size_t)T_cap * DH;

    const int t_first = pad ? (int)min((int64_t)step, max((int64_t)0, pad[b])) : 0;
    const int span = step - t_first;
    const int per = (span + nsplit - 1) / nsplit;
    const int t0 = t_first + split * per;
    const int t1 = min(step, t0 + per);
    const int n = max(0, t1 - t0);

    // Append the new token's k, v (row step-1).  The workgroup that owns that
    // row keeps it in registers for its own use (every lane holds the slice
    // `sub` of the new k and v) and writes it to the cache on the side; no
    // other workgroup of this launch reads that row, so no fence is needed.
    // With a rotary row given, k is rotated on the way in (pairs d, d + DH/2).
    const bool own_last = k_new != nullptr && step - 1 >= t0 && step - 1 < t1;
    u32x4 knew = {0, 0, 0, 0}, vnew = {0, 0, 0, 0};
    if (own_last) {
        knew = *reinterpret_cast<const u32x4 *>(k_new + qoff + sub * 8);
        if (rope_row != nullptr) {
            const u32x4 ky = *reinterpret_cast<const u32x4 *>(k_new + qoff + (sub ^ (LPR / 2)) * 8);
            knew = rotate8<DH>(knew, ky, sub, rope_row);
        }
        vnew = *reinterpret_cast<const u32x4 *>(v_new + qoff + sub * 8);
        if (rs == 0) {
            *reinterpret_cast<u32x4 *>(kc + (size_t)(step - 1) * DH + sub * 8) = knew;
            *reinterpret_cast<u32x4 *>(vc + (size_t)(step - 1) * DH + sub * 8) = vnew;
        }
    }
    const int r_last = own_last ? step - 1 - t0 : -1;

    u32x4 qv = *reinterpret_cast<const u32x4 *>(q + qoff + sub * 8);
    if (rope_row != nullptr) {
        u32x4 qy;
        qy.x = __shfl_xor(qv.x, LPR / 2, 64);
        qy.y = __shfl_xor(qv.y, LPR / 2, 64);
        qy.z = __shfl_xor(qv.z, LPR / 2, 64);
        qy.w = __shfl_xor(qv.w, LPR / 2, 64);
        qv = rotate8<DH>(qv, qy, sub, rope_row);
    }

    // Every group of LPR lanes walks its own stream of rows (rs, rs + RPB, ...)
    // with a running softmax (max m, sum l, un-normalised acc): K and V rows are
    // requested together, UN rows deep, and nothing synchronises the workgroup
    // until the streams are merged at the end.
    float m_run = -INFINITY, l_run = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int r0 = rs; r0 < n; r0 += RPB * UN) {
        u32x4 kv[UN], vv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int r = r0 + u * RPB;
            if (r < n)
                kv[u] = (r == r_last)
                            ? knew
                            : load_row16(reinterpret_cast<const u32x4 *>(kc + (size_t)(t0 + r) * DH) + sub);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int r = r0 + u * RPB;
            if (r < n)
                vv[u] = (r == r_last)
                            ? vnew
                            : load_row16(reinterpret_cast<const u32x4 *>(vc + (size_t)(t0 + r) * DH) + sub);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int r = r0 + u * RPB;  // the same for all LPR lanes of a group
            float d = (r < n) ? dot8(qv, kv[u]) : 0.f;
            d = group_sum<LPR>(d) * scale;
            if (r < n) {
                if (alibi)
                    d += (float)alibi[(size_t)h * alibi_ld + t0 + r];
                const float m_new = fmaxf(m_run, d);
                const float c = __expf(m_run - m_new);  // 0 on the first row (m_run = -inf)
                const float p = __expf(d - m_new);
                l_run = l_run * c + p;
                const half8 hv = __builtin_bit_cast(half8, vv[u]);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    acc[e] = acc[e] * c + p * (float)hv[e];
                m_run = m_new;
            }
        }
    }

    // Merge the RPB streams of the workgroup.
#pragma unroll
    for (int e = 0; e < 8; ++e)
        accs[rs][sub * 8 + e] = acc[e];
    if (sub == 0) {
        stream_m[rs] = m_run;
        stream_l[rs] = l_run;
    }
    __syncthreads();
    if (tid < DH) {
        float lmax = -INFINITY;
#pragma unroll 4
        for (int r = 0; r < RPB; ++r)
            lmax = fmaxf(lmax, stream_m[r]);
        float s = 0.f, lsum = 0.f;
#pragma unroll 4
        for (int r = 0; r < RPB; ++r) {
            const float mr = stream_m[r];
            const float w = (mr == -INFINITY) ? 0.f : __expf(mr - lmax);
            lsum += w * stream_l[r];
            s += w * accs[r][tid];
        }
        if (nsplit == 1) {
            // n == 0 (everything padded away) gives 0 / 1e-6 = 0.
            ctx[coff + tid] = (_Float16)(s / (lsum + 1e-6f));
        } else {
            float *p = partial + ((size_t)bh * nsplit + split) * (DH + 2);
            p[2 + tid] = s;
            if (tid == 0) {
                p[0] = lmax;
                p[1] = lsum;
            }
        }
    }
}

template <int DH>
__global__ __launch_bounds__(DH) void mmha_decode_merge_kernel(const float *__restrict__ partial,
                                                               _Float16 *__restrict__ ctx, int nsplit)
{
    const int bh = blockIdx.x, tid = threadIdx.x;
    const float *p = partial + (size_t)bh * nsplit * (DH + 2);
    float m = -INFINITY;
    for (int s = 0; s < nsplit; ++s)
        m = fmaxf(m, p[s * (DH + 2)]);
    float sum = 0.f, acc = 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float ms = p[s * (DH + 2)];
        const float w = (ms == -INFINITY) ? 0.f : __expf(ms - m);
        sum += w * p[s * (DH + 2) + 1];
        acc += w * p[s * (DH + 2) + 2 + tid];
    }
    ctx[(size_t)bh * DH + tid] = (_Float16)(acc / (sum + 1e-6f));
}

int pick_nsplit(int BH, int step)
{
    static const int forced = [] {
        const char *e = std::getenv("EET_MMHA_NSPLIT");  // tuning override
        return e ? atoi(e) : 0;
    }();
    if (forced > 0)
        return forced;
    // Measured on MI355X (B*H = 256 at step ~1100 and B*H = 1280 at step ~2200):
    // up to ~4096 workgroups, but no fewer than 256 rows each.
    int want = (4096 + BH - 1) / BH;
    int by_rows = step / 256;
    int ns = want < by_rows ? want : by_rows;
    return ns < 1 ? 1 : ns;
}

template <int DH>
int launch(const void *q, const void *k, const void *v, long qkv_stride, void *kc, void *vc, void *ctx,
           const void *alibi, const int64_t *pad, int B, int H, int step, int T_cap, void *ws, int nsplit,
           const float *rope_row, hipStream_t st)
{
    const float scale = (float)(_Float16)(1.0f / sqrtf((float)DH));
    dim3 grid(B * H, nsplit);
    static const int unroll = [] {
        const char *e = std::getenv("EET_MMHA_UNROLL");
        return e ? atoi(e) : 8;
    }();
    auto kern = (unroll == 4) ? mmha_decode_split_kernel<DH, 4> : mmha_decode_split_kernel<DH, 8>;
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), 0, st,
                       static_cast<const _Float16 *>(q), static_cast<const _Float16 *>(k),
                       static_cast<const _Float16 *>(v), qkv_stride, static_cast<_Float16 *>(kc),
                       static_cast<_Float16 *>(vc), static_cast<_Float16 *>(ctx),
                       static_cast<const _Float16 *>(alibi), pad, static_cast<float *>(ws), H, step, T_cap, nsplit,
                       scale, rope_row);
    EET_HIP_CHECK(hipGetLastError());
    if (nsplit > 1) {
        hipLaunchKernelGGL((mmha_decode_merge_kernel<DH>), dim3(B * H), dim3(DH), 0, st,
                           static_cast<const float *>(ws), static_cast<_Float16 *>(ctx), nsplit);
        EET_HIP_CHECK(hipGetLastError());
    }
    return EET_OK;
}

}  // namespace

namespace {
// table[t][i] = cos(t / 10000^(2i/dh)), table[t][dh/2 + i] = sin(...), fp32
// (csrc/core/common.cuh:176-180).
__global__ void rope_table_kernel(float *table, int T, int dh)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= T * (dh / 2))
        return;
    const int t = idx / (dh / 2), i = idx % (dh / 2);
    const float ang = (float)t / powf(10000.0f, (float)(2 * i) / (float)dh);
    table[(size_t)t * dh + i] = cosf(ang);
    table[(size_t)t * dh + dh / 2 + i] = sinf(ang);
}
}  // namespace

extern "C" int eet_rope_table(float *table, int T, int dh, void *stream)
{
    EET_REQUIRE(table != nullptr, EET_ERR_INVALID_ARGUMENT, "eet_rope_table: null pointer");
    EET_REQUIRE(T > 0 && dh > 0 && dh % 2 == 0, EET_ERR_INVALID_ARGUMENT, "eet_rope_table: bad sizes T=%d dh=%d", T, dh);
    const int n = T * (dh / 2);
    hipLaunchKernelGGL(rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), table,
                       T, dh);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" size_t eet_mmha_decode_workspace(int B, int H, int dh, int step)
{
    if (B <= 0 || H <= 0 || dh <= 0 || step <= 0)
        return 0;
    const int ns = pick_nsplit(B * H, step);
    return ns > 1 ? (size_t)B * H * ns * (dh + 2) * sizeof(float) : 0;
}

extern "C" int eet_mmha_decode(const void *q, const void *k, const void *v, long qkv_stride, void *k_cache,
                               void *v_cache, void *ctx, const void *alibi, const int64_t *pad, int B, int H,
                               int dh, int step, int T_cap, const float *rope_cos_sin, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    EET_REQUIRE(q && k_cache && v_cache && ctx, EET_ERR_INVALID_ARGUMENT, "eet_mmha_decode: null pointer");
    EET_REQUIRE((k == nullptr) == (v == nullptr), EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_decode: k and v must both be given or both be NULL");
    EET_REQUIRE(B > 0 && H > 0 && step > 0 && T_cap > 0, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_decode: bad sizes B=%d H=%d step=%d T_cap=%d", B, H, step, T_cap);
    EET_REQUIRE(step <= T_cap, EET_ERR_INVALID_ARGUMENT, "eet_mmha_decode: step %d exceeds the cache capacity %d",
                step, T_cap);
    EET_REQUIRE(dh == 32 || dh == 64 || dh == 128, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_mmha_decode: head size %d not supported (32, 64, 128)", dh);
    EET_REQUIRE(qkv_stride >= 0 && qkv_stride % 8 == 0, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_decode: qkv_stride must be a non-negative multiple of 8");
    EET_REQUIRE(rope_cos_sin == nullptr || k != nullptr, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_decode: a rotary row needs the new k, v (it rotates q and the appended k)");
    const int ns = pick_nsplit(B * H, step);
    const size_t need = eet_mmha_decode_workspace(B, H, dh, step);
    EET_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), EET_ERR_WORKSPACE,
                "eet_mmha_decode: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dh) {
        case 32:
            return launch<32>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, workspace,
                              ns, rope_cos_sin, st);
        case 64:
            return launch<64>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, workspace,
                              ns, rope_cos_sin, st);
        default:
            return launch<128>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap,
                               workspace, ns, rope_cos_sin, st);
    }
}
