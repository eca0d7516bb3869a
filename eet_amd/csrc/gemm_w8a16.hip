// Fused dequant-GEMM: C[M][N] = A[M][K] (fp16) . (int8 W[K][N] * scale[N]).
//
// Replaces fastertransformer::gemm_fp16_int_bias_act<uint8_t>
// (3rdparty/cutlass_kernels/fpA_intB_gemm.cu:35-62) as EET calls it: no bias,
// no activation, no split-K workspace (csrc/op/llama_mmha.cpp:313-337).
//
// Weights arrive in the gfx950 layout written by eet_pack_gfx950: 1 KiB tiles
// of 16 output channels x 64 input features, tile order [n_tile][k_tile], lane
// l = 16*g + i of a wavefront owns bytes [16*l, 16*l+16) = channel i, features
// 16*g .. 16*g+15 of the tile, each stored as q + 128.
//
// Small-M kernel (M <= 32, HBM-bound).  A workgroup owns NT n-tiles over the
// whole K range; its wavefronts take k-tiles round-robin, so the workgroup
// streams one contiguous byte range per n-tile with one 128-bit load per lane
// per tile.  A tile is widened to fp16 in registers (byte-permute into
// 0x6400|u8, packed subtract of 1152) and fed to v_mfma_f32_16x16x32_f16 as the
// 16x32 operand; the activations are the 32x16 operand, read straight from
// global memory (they are tiny and live in L2) and reused for all NT tiles.
// The matrix core is used because the vector ALU cannot keep up with HBM here:
// 8 TB/s of int8 weights at M = 16 needs 256 TFLOP/s of multiply-adds plus the
// widening, above the chip's vector-fp32 peak, but only ~10 % of its fp16 MFMA
// peak.  Partial sums of the wavefronts meet in LDS; the per-channel scale is
// applied once to the fp32 sum (the reference multiplies every weight by the
// scale in fp16 first, mma_tensorop_dequantizer.h:258-275 -- this is strictly
// more accurate and inside the 1e-2 / 1e-3 tolerance against fp32).
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 4 biased bytes -> 4 fp16 values (q = u8 - 128), exact.
__device__ __forceinline__ void widen4(uint32_t x, half2v &lo, half2v &hi)
{
    const half2v magic = {(_Float16)1152.0f, (_Float16)1152.0f};
    uint32_t a = __builtin_amdgcn_perm(0x64646464u, x, 0x04010400u);  // {0x64, b1, 0x64, b0}
    uint32_t b = __builtin_amdgcn_perm(0x64646464u, x, 0x04030402u);  // {0x64, b3, 0x64, b2}
    lo = __builtin_bit_cast(half2v, a) - magic;
    hi = __builtin_bit_cast(half2v, b) - magic;
}

__device__ __forceinline__ half8 widen8(uint32_t x0, uint32_t x1)
{
    half2v a, b, c, d;
    widen4(x0, a, b);
    widen4(x1, c, d);
    half8 r = {a.x, a.y, b.x, b.y, c.x, c.y, d.x, d.y};
    return r;
}

// One batch of U k-tiles: the raw weight tiles of NT n-tiles and the matching
// activation operands of MT m-tiles, as they come back from memory.
template <int NT, int MT, int U>
struct Batch {
    u32x4 w[U][NT];
    u32x4 a[U][MT][2];
};

template <int NT, int MT, int WAVES, int U>
__device__ __forceinline__ void load_batch(Batch<NT, MT, U> &b, const u32x4 *const (&wbase)[NT],
                                           const u32x4 *const (&abase)[MT], int kt)
{
    // All weight loads (HBM latency) go out first, then the activation loads
    // (L2 hits); loads return in issue order.
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            b.w[u][t] = __builtin_nontemporal_load(wbase[t] + (size_t)(kt + u * WAVES) * 64);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            b.a[u][mt][0] = abase[mt][(kt + u * WAVES) * 8];
            b.a[u][mt][1] = abase[mt][(kt + u * WAVES) * 8 + 1];
        }
    __builtin_amdgcn_sched_barrier(0);
}

template <int NT, int MT, int U>
__device__ __forceinline__ void mma_batch(const Batch<NT, MT, U> &b, floatx4 (&acc)[NT][MT])
{
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const half8 w0 = widen8(b.w[u][t].x, b.w[u][t].y);
            const half8 w1 = widen8(b.w[u][t].z, b.w[u][t].w);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, __builtin_bit_cast(half8, b.a[u][mt][0]),
                                                                    acc[t][mt], 0, 0, 0);
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, __builtin_bit_cast(half8, b.a[u][mt][1]),
                                                                    acc[t][mt], 0, 0, 0);
            }
        }
}

template <int NT, int MT, int WAVES, int U>
__global__ __launch_bounds__(WAVES * 64) void w8a16_small_m_kernel(
    const _Float16 *__restrict__ A, const u32x4 *__restrict__ Wp, const _Float16 *__restrict__ scale,
    _Float16 *__restrict__ C, int M, int N, int K)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int g = lane >> 4, j = lane & 15;
    const int ktiles = K >> 6;
    const int ntiles = N >> 4;
    const int nt0 = blockIdx.x * NT;

    floatx4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // A tile index past the end is clamped: its results are never written.
    const u32x4 *wbase[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        int nt = min(nt0 + t, ntiles - 1);
        wbase[t] = Wp + (size_t)nt * ktiles * 64 + lane;
    }
    // Lanes whose row is past M read row M-1: column m of the product depends
    // only on activation row m, and rows >= M are not written.
    const u32x4 *abase[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        int m = min(mt * 16 + j, M - 1);
        abase[mt] = reinterpret_cast<const u32x4 *>(A + (size_t)m * K + 16 * g);
    }

    // This wavefront's k-tiles are wave, wave + WAVES, ...; they are taken in
    // batches of U with the next batch's loads in flight while the current one
    // is multiplied (two register buffers).
    const int mine = (ktiles - wave + WAVES - 1) / WAVES;
    const int nbatch = mine / U;
    constexpr int STEP = U * WAVES;
    int kt = wave;
    {
        Batch<NT, MT, U> b0, b1;
        if (nbatch > 0)
            load_batch<NT, MT, WAVES, U>(b0, wbase, abase, kt);
        int i = 0;
        for (; i + 2 <= nbatch; i += 2) {
            load_batch<NT, MT, WAVES, U>(b1, wbase, abase, kt + STEP);
            mma_batch<NT, MT, U>(b0, acc);
            if (i + 2 < nbatch)
                load_batch<NT, MT, WAVES, U>(b0, wbase, abase, kt + 2 * STEP);
            mma_batch<NT, MT, U>(b1, acc);
            kt += 2 * STEP;
        }
        if (i < nbatch) {
            mma_batch<NT, MT, U>(b0, acc);
            kt += STEP;
        }
    }
    for (; kt < ktiles; kt += WAVES) {
        Batch<NT, MT, 1> b;
        load_batch<NT, MT, WAVES, 1>(b, wbase, abase, kt);
        mma_batch<NT, MT, 1>(b, acc);
    }

    // Per-channel scales for the epilogue, requested before the barrier so
    // their latency overlaps the reduction.
    half4 sc[(NT * MT + WAVES - 1) / WAVES];
    {
        int idx = 0;
        for (int tile = wave; tile < NT * MT; tile += WAVES, ++idx) {
            const int nt = min(nt0 + tile / MT, ntiles - 1);
            sc[idx] = *reinterpret_cast<const half4 *>(scale + nt * 16 + 4 * g);
        }
    }

    // Cross-wavefront reduction.  acc[t][mt][r] of lane (g, j) is the product
    // for channel 16*(nt0+t) + 4*g + r and row 16*mt + j.
    __shared__ floatx4 red[WAVES][NT * MT][64];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            red[wave][t * MT + mt][lane] = acc[t][mt];
    __syncthreads();
    int idx = 0;
    for (int tile = wave; tile < NT * MT; tile += WAVES, ++idx) {
        floatx4 s = red[0][tile][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            s += red[w][tile][lane];
        const int t = tile / MT, mt = tile % MT;
        const int m = mt * 16 + j;
        if (nt0 + t < ntiles && m < M) {
            const int n = (nt0 + t) * 16 + 4 * g;
            half4 o;
            o.x = (_Float16)(s.x * (float)sc[idx].x);
            o.y = (_Float16)(s.y * (float)sc[idx].y);
            o.z = (_Float16)(s.z * (float)sc[idx].z);
            o.w = (_Float16)(s.w * (float)sc[idx].w);
            *reinterpret_cast<half4 *>(C + (size_t)m * N + n) = o;
        }
    }
}

struct SmallMConfig {
    int nt, waves, u;
};

template <int NT, int MT, int WAVES, int U>
int launch_small_m(const void *A, const void *Wp, const void *scale, void *C, int M, int N, int K, hipStream_t st)
{
    const int ntiles = N / 16;
    dim3 grid((ntiles + NT - 1) / NT), block(WAVES * 64);
    hipLaunchKernelGGL((w8a16_small_m_kernel<NT, MT, WAVES, U>), grid, block, 0, st,
                       static_cast<const _Float16 *>(A), static_cast<const u32x4 *>(Wp),
                       static_cast<const _Float16 *>(scale), static_cast<_Float16 *>(C), M, N, K);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

template <int MT>
int dispatch_small_m(SmallMConfig cfg, const void *A, const void *Wp, const void *scale, void *C, int M, int N,
                     int K, hipStream_t st)
{
#define EET_CASE(NT_, W_, U_)                                 \
    if (cfg.nt == NT_ && cfg.waves == W_ && cfg.u == U_)      \
        return launch_small_m<NT_, MT, W_, U_>(A, Wp, scale, C, M, N, K, st);
    EET_CASE(1, 4, 4) EET_CASE(1, 8, 4) EET_CASE(1, 16, 4) EET_CASE(1, 8, 2) EET_CASE(1, 16, 2)
    EET_CASE(2, 4, 2) EET_CASE(2, 8, 2) EET_CASE(2, 16, 2) EET_CASE(2, 8, 4) EET_CASE(2, 16, 1)
    EET_CASE(3, 8, 2) EET_CASE(3, 16, 2) EET_CASE(3, 16, 1) EET_CASE(3, 8, 1)
    EET_CASE(4, 4, 2) EET_CASE(4, 8, 2) EET_CASE(4, 8, 1) EET_CASE(4, 16, 1)
#undef EET_CASE
    return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: no small-M kernel for nt=%d waves=%d u=%d", cfg.nt,
                     cfg.waves, cfg.u);
}

// Shape -> launch shape.  The chip has 256 CUs; aim for a few workgroups per
// CU while keeping every wavefront at least a few k-tiles deep.
SmallMConfig pick_small_m(int M, int N, int K)
{
    const char *env = std::getenv("EET_GEMM_SMALL_M_CONFIG");  // "nt,waves,u": tuning override
    if (env) {
        SmallMConfig c{1, 8, 4};
        if (sscanf(env, "%d,%d,%d", &c.nt, &c.waves, &c.u) == 3)
            return c;
    }
    // Measured on MI355X (LLaMA-7B shapes, M = 1..32): three n-tiles per
    // workgroup reuse each activation operand three times and win whenever
    // that still leaves >= ~200 workgroups; otherwise one n-tile per
    // workgroup, with 16 wavefronts once K is long enough to feed them.
    const int ntiles = N / 16;
    SmallMConfig c;
    if (ntiles >= 600) {
        c = SmallMConfig{3, 8, 1};
    } else if (ntiles >= 400) {
        c = SmallMConfig{2, 8, 2};
    } else if (K >= 8192 && M <= 16) {
        c = SmallMConfig{1, 16, 2};
    } else {
        c = SmallMConfig{1, 8, 2};
    }
    (void)M;
    return c;
}

}  // namespace

int eet_gemm_w8a16_large_m(const void *A, const void *Wp, const void *scale, void *C, int M, int N, int K,
                           hipStream_t st);

extern "C" int eet_gemm_w8a16(const void *A, const void *Wpacked, const void *scale, void *C, int M, int N, int K,
                              void *workspace, size_t workspace_bytes, void *stream)
{
    (void)workspace;
    (void)workspace_bytes;
    EET_REQUIRE(A && Wpacked && scale && C, EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: null pointer");
    EET_REQUIRE(M >= 0 && N > 0 && K > 0, EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: bad sizes M=%d N=%d K=%d", M,
                N, K);
    EET_REQUIRE(K % 64 == 0 && N % 16 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_gemm_w8a16: need K %% 64 == 0 and N %% 16 == 0, got K=%d N=%d", K, N);
    EET_REQUIRE((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Wpacked)) % 16 == 0 &&
                    (reinterpret_cast<uintptr_t>(scale) | reinterpret_cast<uintptr_t>(C)) % 8 == 0,
                EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: A and W must be 16-byte aligned, scale and C 8-byte");
    if (M == 0)
        return EET_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (M <= 32) {
        SmallMConfig cfg = pick_small_m(M, N, K);
        if (M <= 16)
            return dispatch_small_m<1>(cfg, A, Wpacked, scale, C, M, N, K, st);
        return dispatch_small_m<2>(cfg, A, Wpacked, scale, C, M, N, K, st);
    }
    return eet_gemm_w8a16_large_m(A, Wpacked, scale, C, M, N, K, st);
}

// Interim large-M path: the small-M kernel over 32-row slabs (re-reads the
// weights once per slab).
int eet_gemm_w8a16_large_m(const void *A, const void *Wp, const void *scale, void *C, int M, int N, int K,
                           hipStream_t st)
{
    SmallMConfig cfg = pick_small_m(32, N, K);
    for (int m0 = 0; m0 < M; m0 += 32) {
        const int mm = (M - m0 < 32) ? M - m0 : 32;
        const _Float16 *a = static_cast<const _Float16 *>(A) + (size_t)m0 * K;
        _Float16 *c = static_cast<_Float16 *>(C) + (size_t)m0 * N;
        int rc = (mm <= 16) ? dispatch_small_m<1>(cfg, a, Wp, scale, c, mm, N, K, st)
                            : dispatch_small_m<2>(cfg, a, Wp, scale, c, mm, N, K, st);
        if (rc)
            return rc;
    }
    return EET_OK;
}
