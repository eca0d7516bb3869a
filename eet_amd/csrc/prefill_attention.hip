// Causal prompt attention as one flash-style kernel on the fp16 MFMA units.
//
// Replaces the reference's unfused prompt pass -- cuBLAS QK^T into a
// [B][H][S][S] buffer, softmax_kernel / masked_softmax_kernel over it, cuBLAS
// P.V and a transpose (csrc/op/llama_mmha.cpp:160-186, csrc/op/
// baichuan_mmha.cpp:120-150, csrc/core/gpt2_self_softmax.cu:8-258) -- without
// ever materialising S x S and without the reference's S <= 2048 / 4096 limits.
// Semantics kept: logits = (q . k) * half(1/sqrt(dh)) [+ slope_h * j], keys
// j > i and j < pad[b] masked, denominator + 1e-6, query rows i < pad[b] give
// zeros; fp32 softmax statistics and accumulation, probabilities rounded to
// fp16 for the second MFMA.
//
// Everything is computed transposed so that one lane owns one query:
//   S^T[key][q] = K . Q^T   (A operand = K rows from LDS, B operand = Q^T in registers)
//   O^T[d][q]  += V^T . P^T (A operand = V^T from LDS,   B operand = P^T, already in place)
// With v_mfma_f32_16x16x32_f16 the result lane (g, j) holds column j (= query)
// and rows 4g..4g+3, so the running max / sum / rescale of a query are
// per-lane scalars, and the fp16 P^T operand of the second product is exactly
// the first product's output registers (the 32 contraction slots of a lane
// group g are keys 4g..4g+3 of two adjacent 16-key tiles; V^T is read from LDS
// in the same slot order).
//
// A workgroup of 4 wavefronts takes 128 queries of one (b, h) (32 per
// wavefront) and walks the keys in chunks of 64.  K rows go to LDS as they are
// (row stride padded by 16 bytes); V is transposed on its way into LDS (each
// thread loads 4 keys x 8 d and stores eight 4-key groups) with an XOR swizzle
// that keeps both the stores and the operand reads bank-conflict free.  The
// next chunk is prefetched into registers while the current one is multiplied.
#include <hip/hip_runtime.h>

#include <cmath>

#include "common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kBQ = 128;   // queries per workgroup
constexpr int kBK = 64;    // keys per chunk
constexpr int kQT = 2;     // 16-query tiles per wavefront

__device__ __forceinline__ int vt_swizzle(int d) { return (d & 15) ^ ((d >> 3) & 15); }

template <int DH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void prefill_attention_kernel(
    const _Float16 *__restrict__ q, const _Float16 *__restrict__ k_cache, const _Float16 *__restrict__ v_cache,
    _Float16 *__restrict__ ctx, const _Float16 *__restrict__ alibi, const int64_t *__restrict__ pad, int H, int S,
    int T_cap, float scale)
{
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    constexpr int DC = DH / 32;            // 32-wide d chunks of the first product
    constexpr int DT = DH / 16;            // 16-row d tiles of the second product
    constexpr int KROW = DH * 2 + 16;      // bytes per K row in LDS
    constexpr int PPR = DH / 8;            // 16-byte pieces per row
    constexpr int K_ITEMS = kBK * PPR / kThreads > 0 ? kBK * PPR / kThreads : 1;
    __shared__ __attribute__((aligned(16))) unsigned char lds_k[kBK * KROW];
    __shared__ __attribute__((aligned(16))) _Float16 lds_vt[DH * kBK];  // [d][16 key groups of 4], swizzled

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, j = lane & 15;
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    const int q_blocks = (S + kBQ - 1) / kBQ;
    const int q0 = (q_blocks - 1 - (int)blockIdx.x) * kBQ;  // late (long) query blocks first
    const int padb = pad ? (int)min((int64_t)S, max((int64_t)0, pad[b])) : 0;

    const _Float16 *kbase = k_cache + (size_t)bh * T_cap * DH;
    const _Float16 *vbase = v_cache + (size_t)bh * T_cap * DH;
    const _Float16 *qbase = q + (size_t)bh * S * DH;

    // Q^T operands: lane (g, j) holds d = 32c + 8g .. +7 of query wq0 + 16*qt + j
    const int wq0 = q0 + wave * (16 * kQT);
    half8 qop[kQT][DC];
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        const int qi = min(wq0 + 16 * qt + j, S - 1);
#pragma unroll
        for (int c = 0; c < DC; ++c)
            qop[qt][c] = *reinterpret_cast<const half8 *>(qbase + (size_t)qi * DH + 32 * c + 8 * g);
    }

    floatx4 oacc[kQT][DT];
    float m_run[kQT], l_run[kQT];
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        m_run[qt] = -INFINITY;
        l_run[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            oacc[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // staging registers: K pieces (row-wise) and a 4-key x 8-d block of V per item
    constexpr int V_ITEMS = (16 * PPR + kThreads - 1) / kThreads;
    u32x4 kreg[K_ITEMS], vreg[V_ITEMS][4];
    auto load_chunk = [&](int kc0) {
#pragma unroll
        for (int it = 0; it < K_ITEMS; ++it) {
            const int piece = tid + it * kThreads;
            if (piece < kBK * PPR) {
                const int key = min(kc0 + piece / PPR, S - 1);
                kreg[it] = *reinterpret_cast<const u32x4 *>(kbase + (size_t)key * DH + (piece % PPR) * 8);
            }
        }
#pragma unroll
        for (int it = 0; it < V_ITEMS; ++it) {
            const int item = tid + it * kThreads;
            if (item < 16 * PPR) {
                const int kg = item / PPR, p = item % PPR;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = min(kc0 + 4 * kg + r, S - 1);
                    vreg[it][r] = *reinterpret_cast<const u32x4 *>(vbase + (size_t)key * DH + p * 8);
                }
            }
        }
    };
    auto store_chunk = [&]() {
#pragma unroll
        for (int it = 0; it < K_ITEMS; ++it) {
            const int piece = tid + it * kThreads;
            if (piece < kBK * PPR)
                *reinterpret_cast<u32x4 *>(lds_k + (piece / PPR) * KROW + (piece % PPR) * 16) = kreg[it];
        }
#pragma unroll
        for (int it = 0; it < V_ITEMS; ++it) {
            const int item = tid + it * kThreads;
            if (item < 16 * PPR) {
                const int kg = item / PPR, p = item % PPR;
                half8 rows[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    rows[r] = __builtin_bit_cast(half8, vreg[it][r]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int d = 8 * p + e;
                    half4 col = {rows[0][e], rows[1][e], rows[2][e], rows[3][e]};
                    *reinterpret_cast<half4 *>(lds_vt + d * kBK + ((kg ^ vt_swizzle(d)) * 4)) = col;
                }
            }
        }
    };

    const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(alibi ? alibi + (size_t)h * S : q), 0, alibi ? (unsigned)S * 2u : 0u, 0x00020000);
    const bool bias_wide = (S % 4 == 0) && (reinterpret_cast<uintptr_t>(alibi) % 8 == 0);
    // exponentials are taken as 2^x: log2(e) is folded into the logit scale and the bias
    constexpr float kLog2e = 1.4426950408889634f;
    const float scale2 = scale * kLog2e;
    const int k_begin = (padb / kBK) * kBK;
    const int k_end = min(S, q0 + kBQ);  // keys beyond the block's last query are never needed
    if (k_begin < k_end)
        load_chunk(k_begin);
    for (int kc0 = k_begin; kc0 < k_end; kc0 += kBK) {
        __syncthreads();  // previous chunk fully consumed
        store_chunk();
        __syncthreads();
        // ALiBi terms of this chunk's keys (keys kc0 + 16*kt + 4g .. +3 are 8 contiguous bytes; reads
        // past the table return zero, those keys are masked anyway), requested before the prefetch
        // below: loads return in order, so asking for them later would mean waiting for the whole
        // next chunk as well
        half4 bias4[4];
        if (bias_wide) {
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                bias4[kt] = __builtin_bit_cast(
                    half4, __builtin_amdgcn_raw_buffer_load_b64(ars, (unsigned)((kc0 + 16 * kt + 4 * g) * 2), 0, 0));
        } else {  // a head's row of the table is not 8-byte aligned (S % 4 != 0): element loads
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    bias4[kt][r] = __builtin_bit_cast(
                        _Float16, __builtin_amdgcn_raw_buffer_load_b16(ars, (unsigned)((kc0 + 16 * kt + 4 * g + r) * 2), 0, 0));
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kc0 + kBK < k_end)
            load_chunk(kc0 + kBK);

        // a wavefront whose queries all precede this chunk has nothing to do in it
        if (kc0 > wq0 + 16 * kQT - 1)
            continue;

        // S^T = K . Q^T for the 4 key tiles of the chunk
        floatx4 sacc[kQT][4];
#pragma unroll
        for (int qt = 0; qt < kQT; ++qt)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                sacc[qt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                const half8 kop = *reinterpret_cast<const half8 *>(lds_k + (16 * kt + j) * KROW + (4 * c + g) * 16);
#pragma unroll
                for (int qt = 0; qt < kQT; ++qt)
                    sacc[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, qop[qt][c], sacc[qt][kt], 0, 0, 0);
            }
        }

        // online softmax; lane (g, j) holds keys kc0 + 16*kt + 4g + r of query wq0 + 16*qt + j
        half8 pop[kQT][2];
#pragma unroll
        for (int qt = 0; qt < kQT; ++qt) {
            const int qi = wq0 + 16 * qt + j;
            float cmax = -INFINITY;
            // only chunks that touch the diagonal or the padded prefix need the mask
            const bool need_mask = (kc0 + kBK - 1 > wq0) || (kc0 < padb);
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float s = sacc[qt][kt][r] * scale2 + (float)bias4[kt][r] * kLog2e;
                    if (need_mask) {
                        const int key = kc0 + 16 * kt + 4 * g + r;
                        s = (key > qi || key < padb) ? -INFINITY : s;
                    }
                    sacc[qt][kt][r] = s;
                    cmax = fmaxf(cmax, s);
                }
            cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
            cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
            const float m_new = fmaxf(m_run[qt], cmax);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float corr = __builtin_amdgcn_exp2f(m_run[qt] - m_safe);  // 0 while nothing has been seen
            float psum = 0.f;
            float p[4][4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    p[kt][r] = __builtin_amdgcn_exp2f(sacc[qt][kt][r] - m_safe);
                    psum += p[kt][r];
                }
            l_run[qt] = l_run[qt] * corr + psum;  // per-lane share; lanes of a query are summed at the end
            m_run[qt] = m_new;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                oacc[qt][dt] *= corr;
            // P^T operands: contraction slots of lane group g = keys 4g..4g+3 of tile 2*hf, then of tile 2*hf+1
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                half8 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o[r] = (_Float16)p[2 * hf][r];
                    o[4 + r] = (_Float16)p[2 * hf + 1][r];
                }
                pop[qt][hf] = o;
            }
        }

        // O^T += V^T . P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int d = 16 * dt + j;
            const int sw = vt_swizzle(d);
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                // keys 32*hf + 4g .. +3 (key group 8*hf + g) and 32*hf + 16 + 4g .. +3 (key group 8*hf + 4 + g)
                const half4 lo = *reinterpret_cast<const half4 *>(lds_vt + d * kBK + (((8 * hf + g) ^ sw) * 4));
                const half4 hi = *reinterpret_cast<const half4 *>(lds_vt + d * kBK + (((8 * hf + 4 + g) ^ sw) * 4));
                const half8 vop = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int qt = 0; qt < kQT; ++qt)
                    oacc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vop, pop[qt][hf], oacc[qt][dt], 0, 0, 0);
            }
        }
    }

    // normalise and write: lane (g, j) holds d = 16*dt + 4g + r of query wq0 + 16*qt + j
#pragma unroll
    for (int qt = 0; qt < kQT; ++qt) {
        float l = l_run[qt];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        const int qi = wq0 + 16 * qt + j;
        if (qi >= S)
            continue;
        const float inv = (qi < padb) ? 0.f : 1.0f / (l + 1e-6f);
        _Float16 *dst = ctx + ((size_t)(b * S + qi) * H + h) * DH;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            half4 o;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                o[r] = (_Float16)(oacc[qt][dt][r] * inv);
            *reinterpret_cast<half4 *>(dst + 16 * dt + 4 * g) = o;
        }
    }
#endif
}

template <int DH>
int launch(const void *q, const void *kc, const void *vc, void *ctx, const void *alibi, const int64_t *pad, int B,
           int H, int S, int T_cap, hipStream_t st)
{
    const float scale = (float)(_Float16)(1.0f / sqrtf((float)DH));
    dim3 grid((S + kBQ - 1) / kBQ, B * H);
    hipLaunchKernelGGL((prefill_attention_kernel<DH>), grid, dim3(kThreads), 0, st, static_cast<const _Float16 *>(q),
                       static_cast<const _Float16 *>(kc), static_cast<const _Float16 *>(vc),
                       static_cast<_Float16 *>(ctx), static_cast<const _Float16 *>(alibi), pad, H, S, T_cap, scale);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

}  // namespace

extern "C" int eet_prefill_attention(const void *q, const void *k_cache, const void *v_cache, void *ctx,
                                     const void *alibi, const int64_t *pad, int B, int H, int S, int dh, int T_cap,
                                     void *stream)
{
    EET_REQUIRE(q && k_cache && v_cache && ctx, EET_ERR_INVALID_ARGUMENT, "eet_prefill_attention: null pointer");
    EET_REQUIRE(B > 0 && H > 0 && S > 0 && S <= T_cap, EET_ERR_INVALID_ARGUMENT,
                "eet_prefill_attention: bad sizes B=%d H=%d S=%d T_cap=%d", B, H, S, T_cap);
    EET_REQUIRE(dh == 32 || dh == 64 || dh == 96 || dh == 128, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_prefill_attention: head size %d not supported (32, 64, 96, 128)", dh);
    EET_REQUIRE((long long)B * H <= 65535, EET_ERR_UNSUPPORTED_SHAPE, "eet_prefill_attention: B*H too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dh) {
        case 32: return launch<32>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        case 64: return launch<64>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        case 96: return launch<96>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        default: return launch<128>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
    }
}
