// Pieces shared by the small-M (HBM-bound) and large-M (MFMA-bound) dequant-GEMM
// kernels: vector types, the exact int8 -> fp16 widening, epilogue codes and the
// argument block the dispatcher hands to the launchers.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace eet {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

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

// Epilogues: plain; + residual[M][N] (fp16 add); SwiGLU over (gate, up) n-tile
// pairs of an interleaved weight, output [M][N/2].
constexpr int kEpiNone = 0, kEpiResidual = 1, kEpiSwiglu = 2;

struct GemmArgs {
    const _Float16 *A;
    const u32x4 *Wp;
    const _Float16 *scale;
    _Float16 *C;
    int M, N, K;
    const _Float16 *residual;
    int epi;
    const _Float16 *rms_gamma;  // non-null: RMSnorm prologue (small-M kernel only)
    float rms_eps;
    void *ws;  // optional fp32 workspace (split-k partial results)
    size_t ws_bytes;
    hipStream_t st;
    int chain = 0;  // kChainOff / kChainFirst / kChainNext (chain.h; small-M kernel only)
};

// gemm_w8a16_large.hip: the MFMA-tile kernel for M > 32, and the workspace it can use.
int run_large_m(const GemmArgs &a);
size_t large_m_workspace(int M, int N, int K, int epi);

}  // namespace eet
