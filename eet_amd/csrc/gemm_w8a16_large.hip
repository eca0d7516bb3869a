// Large-M fused dequant-GEMM (M > 32 apart from the 32-row-slab case; prefill;
// fp16-MFMA bound).
//
// Replaces the tensor-core side of fastertransformer::gemm_fp16_int_bias_act<uint8_t>
// (3rdparty/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h:48-177).
//
// A workgroup of WNW wavefronts side by side owns a block tile of TM*16 rows x
// WNW*TN*16 channels; each wavefront owns TM x TN tiles of
// v_mfma_f32_16x16x32_f16 (TM*TN*4 fp32 accumulator registers).  What bounds
// such a kernel on a CU is the LDS port (128 B/clk) against the matrix cores
// (4 x 1024 flop/clk): a wavefront tile of WM x WN outputs needs (WM + WN) * 2 B
// of operands per k for 2 * WM * WN flop, so wavefront tiles are made large
// (128 x 64 where M allows) and only one operand goes through LDS:
//   weights      every wavefront reads its own TN packed tiles straight from
//                global memory into registers, two k-tiles ahead -- the packed
//                layout is already the MFMA operand layout -- and widens them
//                once per k-tile;
//   activations  the block's rows x 64 slab is copied global -> LDS by the
//                memory pipeline itself (buffer_load_dwordx4 ... lds: no
//                staging registers, no ds_write) into a ring of four k-tile
//                stages, three tiles ahead of the one being multiplied, and
//                read from there by every wavefront.
// One wavefront row per workgroup, so that two (or more) workgroups share a CU
// with independent barriers; a 256 x 256 block of eight wavefronts with one
// barrier measured 5-10 % slower than two 128 x 256 blocks.  Workgroups are
// numbered so that the ones sharing a weight column block run on the same XCD
// (workgroup i lands on XCD i % 8) and hit its L2.
//
// A stage holds TM m-tiles of 2 KiB: [row half b][row r (8)][position (8)] x
// 16 B, where position p of row (b, r) holds piece p ^ ((r >> 1) | (b << 2)) of
// the row's eight 16-byte pieces.  One DMA instruction fills 1 KiB (8 rows x
// 128 B, whole cache lines; the XOR only permutes lanes within a line), and the
// MFMA operand read of lane (g, j) -- piece 2g+h of row j -- hits 16 distinct
// 16-byte bank groups per 16 lanes.
#include <cstdlib>

#include "gemm_common.h"

using namespace eet;

namespace {

constexpr int kDmaStages = 4, kDmaAhead = 3;

__device__ __forceinline__ constexpr int vmcnt_imm(int n)
{
    return (n & 15) | (7 << 4) | (15 << 8) | ((n >> 4) << 14);  // expcnt, lgkmcnt: no wait
}

template <int WNW, int TM, int TN>
struct DmaShape {
    static constexpr int kThreads = 64 * WNW;
    static constexpr int kBM = TM * 16, kBN = WNW * TN * 16;
    static constexpr int kStageVec = TM * 128;          // u32x4 per stage
    static constexpr int kRowGroups = TM * 2;           // DMA instructions per k-tile (8 rows each)
    static constexpr int kPerWave = kRowGroups / WNW;   // ... per wavefront
    static_assert(kRowGroups % WNW == 0, "row groups must divide over the wavefronts");
    static_assert(kDmaStages * kStageVec * 16 <= 65536, "the stage ring must fit 64 KiB");
};

template <int WNW, int TM, int TN>
__global__ __launch_bounds__(64 * WNW) __attribute__((amdgpu_waves_per_eu(2))) void w8a16_large_m_kernel(
    const _Float16 *__restrict__ A, const u32x4 *__restrict__ Wp, const _Float16 *__restrict__ scale,
    _Float16 *__restrict__ C, int M, int N, int K, int m_blocks, int n_blocks,
    const _Float16 *__restrict__ residual, int epi)
{
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    using S = DmaShape<WNW, TM, TN>;
    // one array per stage: the compiler tells them apart when it places waits
    // between the DMA writes and the LDS reads
    __shared__ u32x4 st0[S::kStageVec], st1[S::kStageVec], st2[S::kStageVec], st3[S::kStageVec];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: feeds scalar offsets and M0
    const int g = lane >> 4, j = lane & 15;
    const int ktiles = K >> 6, ntiles = N >> 4;

    const int total = m_blocks * n_blocks;
    const int per_xcd = (total + 7) / 8;
    const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (tile >= total)
        return;
    const int n_blk = tile / m_blocks, m_blk = tile % m_blocks;
    const int m0 = m_blk * S::kBM;
    const int nt0 = n_blk * (WNW * TN) + wave * TN;

    // Both operands are addressed through buffer resources: a 32-bit lane offset
    // plus a scalar offset per tile, and reads past the end (rows >= M, n-tiles
    // >= N/16) return zeros instead of needing clamped addresses.
    const size_t a_bytes = (size_t)(M - m0) * K * 2;
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(A + (size_t)m0 * K), 0, a_bytes > 0xffffffffull ? 0xffffffffu : (unsigned)a_bytes,
        0x00020000);
    const __amdgpu_buffer_rsrc_t wrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4 *>(Wp), 0, (unsigned)((size_t)K * N), 0x00020000);
    const int woff = lane * 16;
    unsigned wtile[TN];  // byte offset of the n-tile's first k-tile
#pragma unroll
    for (int t = 0; t < TN; ++t)
        wtile[t] = (unsigned)(nt0 + t) * (unsigned)ktiles * 1024u;

    // DMA source of this lane for row group rg = wave * kPerWave + i: row
    // 8*rg + lane/8, piece (lane%8) ^ swizzle.
    int aoff[S::kPerWave];
#pragma unroll
    for (int i = 0; i < S::kPerWave; ++i) {
        const int rg = wave * S::kPerWave + i, r = lane >> 3, b = rg & 1;
        const int piece = (lane & 7) ^ ((r >> 1) | (b << 2));
        aoff[i] = (8 * rg + r) * K * 2 + piece * 16;
    }
    const int swz = ((j & 7) >> 1) | ((j >> 3) << 2);
    const int rs0 = (j >> 3) * 64 + (j & 7) * 8 + ((2 * g) ^ swz), rs1 = rs0 ^ 1;

    floatx4 acc[TN][TM];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int mt = 0; mt < TM; ++mt)
            acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    u32x4 wraw[2][TN];

    auto dma_tile = [&](u32x4 *stage, int kt) {
#pragma unroll
        for (int i = 0; i < S::kPerWave; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(arsrc, stage + (wave * S::kPerWave + i) * 64, 16, aoff[i], kt * 128,
                                                     0, 0);
    };
    auto load_w = [&](u32x4 (&dst)[TN], int kt) {
#pragma unroll
        for (int t = 0; t < TN; ++t)
            dst[t] = __builtin_bit_cast(
                u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, woff, wtile[t] + (unsigned)kt * 1024u, 0));
    };

    // One k-tile: A from `cur`, raw weights from wb; the DMA for tile kt + 3 goes
    // to `ahead`, the weights of tile kt + 2 replace wb once it is widened.
    auto step = [&](const u32x4 *cur, u32x4 *ahead, u32x4 (&wb)[TN], int kt) {
        dma_tile(ahead, min(kt + kDmaAhead, ktiles - 1));
        __builtin_amdgcn_sched_barrier(0);
        half8 w0[TN], w1[TN];
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            w0[t] = widen8(wb[t].x, wb[t].y);
            w1[t] = widen8(wb[t].z, wb[t].w);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_w(wb, min(kt + 2, ktiles - 1));
        half8 aop[2][2];
        aop[0][0] = __builtin_bit_cast(half8, cur[rs0]);
        aop[0][1] = __builtin_bit_cast(half8, cur[rs1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) {
            if (mt + 1 < TM) {
                aop[(mt + 1) & 1][0] = __builtin_bit_cast(half8, cur[(mt + 1) * 128 + rs0]);
                aop[(mt + 1) & 1][1] = __builtin_bit_cast(half8, cur[(mt + 1) * 128 + rs1]);
            }
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0[t], aop[mt & 1][0], acc[t][mt], 0, 0, 0);
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1[t], aop[mt & 1][1], acc[t][mt], 0, 0, 0);
            }
        }
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) {
            if (mt + 1 < TM)
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // 2 LDS reads
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * TN, 0);  // 2*TN MFMA
        }
        __builtin_amdgcn_sched_barrier(0);
        // The DMA of tile kt+1 (issued two steps ago) must have landed before any
        // wavefront reads it: everything older than the loads of the last two steps
        // (2 x (kPerWave DMA + TN weight loads)), then the barrier.
        // (A plain __syncthreads() would drain every outstanding load here: its
        // release fence waits for all DMA writes, including the ones just issued.)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * (S::kPerWave + TN)) : "memory");
    };

    // prologue: tiles 0..2 into stages 0..2, weights of tiles 0 and 1
    load_w(wraw[0], 0);
    dma_tile(st0, 0);
    load_w(wraw[1], min(1, ktiles - 1));
    dma_tile(st1, min(1, ktiles - 1));
    dma_tile(st2, min(2, ktiles - 1));
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    int kt = 0;
    for (; kt + 4 <= ktiles; kt += 4) {
        step(st0, st3, wraw[0], kt);
        step(st1, st0, wraw[1], kt + 1);
        step(st2, st1, wraw[0], kt + 2);
        step(st3, st2, wraw[1], kt + 3);
    }
    if (kt < ktiles)
        step(st0, st3, wraw[0], kt);
    if (kt + 1 < ktiles)
        step(st1, st0, wraw[1], kt + 1);
    if (kt + 2 < ktiles)
        step(st2, st1, wraw[0], kt + 2);

    // acc[t][mt][r] of lane (g, j): row m0 + 16*mt + j, channel 16*(nt0+t) + 4*g + r
    const int mrow0 = m0 + j;
    if (epi == kEpiSwiglu) {
        if constexpr (TN % 2 == 0) {
#pragma unroll
            for (int t = 0; t < TN; t += 2) {
                if (nt0 + t + 1 >= ntiles)
                    continue;
                const half4 sg = *reinterpret_cast<const half4 *>(scale + (nt0 + t) * 16 + 4 * g);
                const half4 su = *reinterpret_cast<const half4 *>(scale + (nt0 + t + 1) * 16 + 4 * g);
                const int n = ((nt0 + t) / 2) * 16 + 4 * g;
#pragma unroll
                for (int mt = 0; mt < TM; ++mt) {
                    const int m = mrow0 + 16 * mt;
                    if (m < M) {
                        half4 o;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float gate = (float)(_Float16)(acc[t][mt][r] * (float)sg[r]);
                            const float up = (float)(_Float16)(acc[t + 1][mt][r] * (float)su[r]);
                            o[r] = (_Float16)(up * gate / (1.0f + __expf(-gate)));
                        }
                        *reinterpret_cast<half4 *>(C + (size_t)m * (N / 2) + n) = o;
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        if (nt0 + t >= ntiles)
            continue;
        const int n = (nt0 + t) * 16 + 4 * g;
        const half4 sc = *reinterpret_cast<const half4 *>(scale + n);
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) {
            const int m = mrow0 + 16 * mt;
            if (m < M) {
                half4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    o[r] = (_Float16)(acc[t][mt][r] * (float)sc[r]);
                if (epi == kEpiResidual)
                    o = o + *reinterpret_cast<const half4 *>(residual + (size_t)m * N + n);
                *reinterpret_cast<half4 *>(C + (size_t)m * N + n) = o;
            }
        }
    }
#endif
}

template <int WNW, int TM, int TN>
int launch_large_m(const GemmArgs &a)
{
    using S = DmaShape<WNW, TM, TN>;
    const int m_blocks = (a.M + S::kBM - 1) / S::kBM, n_blocks = (a.N + S::kBN - 1) / S::kBN;
    const int grid = ((m_blocks * n_blocks + 7) / 8) * 8;
    hipLaunchKernelGGL((w8a16_large_m_kernel<WNW, TM, TN>), dim3(grid), dim3(S::kThreads), 0, a.st, a.A, a.Wp,
                       a.scale, a.C, a.M, a.N, a.K, m_blocks, n_blocks, a.residual, a.epi);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

struct LargeMConfig {
    int tm, tn;  // m-tiles and n-tiles of 16 per wavefront; the block is tm*16 rows x 4*tn*16 channels
};

// Shape -> tile.  Measured on MI355X (M = 33 .. 8192, LLaMA-7B and Baichuan-13B shapes):
//   128 x 256 (two workgroups per CU) is the fastest tile once it yields a few
//     hundred workgroups;
//   64 x 320 wins when it divides the problem into whole rounds of 512 workgroups
//     where 128 x 256 leaves a CU with two tiles against one elsewhere (M = 2048,
//     N = 5120: 512 tiles, two per CU, instead of 320);
//   64 x 256, 64 x 128 and 32 x 128 keep the chip occupied for M in the tens and
//     hundreds, where the k-loop latency of a few large tiles would dominate.
LargeMConfig pick_large_m(int M, int N, int epi)
{
    auto wgs = [&](int bm, int bn) { return ((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    const int big = wgs(128, 256);
    if (big >= 320) {
        if (epi != kEpiSwiglu) {  // 5 n-tiles per wavefront: no (gate, up) pairs
            // time in units of one 128 x 256 tile on a CU of its own; 64 x 320 is 0.625 of that
            // area and runs at about 0.9 of the large tile's rate
            const double cost_big = 2.0 * ((big + 511) / 512);
            const double cost_320 = 2.0 * ((wgs(64, 320) + 511) / 512) * 0.625 / 0.9;
            if (cost_320 < cost_big)
                return LargeMConfig{4, 5};
        }
        return LargeMConfig{8, 4};
    }
    if (wgs(64, 256) >= 600)
        return LargeMConfig{4, 4};
    if (wgs(64, 128) >= 300)
        return LargeMConfig{4, 2};
    return LargeMConfig{2, 2};
}

}  // namespace

int eet::run_large_m(const GemmArgs &a)
{
    // the kernel addresses A rows and the packed weights with 32-bit byte offsets
    if ((size_t)a.K * a.N >= (1ull << 31) || (size_t)a.K * 2 * 256 >= (1ull << 31))
        return eet::fail(EET_ERR_UNSUPPORTED_SHAPE, "eet_gemm_w8a16: K x N = %d x %d exceeds the 2 GiB weight limit",
                         a.K, a.N);
    LargeMConfig c = pick_large_m(a.M, a.N, a.epi);
    if (const char *env = std::getenv("EET_GEMM_LARGE_M_TILE")) {  // "tm,tn": tuning override
        LargeMConfig e = c;
        if (sscanf(env, "%d,%d", &e.tm, &e.tn) == 2 && (a.epi != kEpiSwiglu || e.tn % 2 == 0))
            c = e;
    }
    if (c.tm == 8 && c.tn == 4)
        return launch_large_m<4, 8, 4>(a);
    if (c.tm == 4 && c.tn == 5)
        return launch_large_m<4, 4, 5>(a);
    if (c.tm == 4 && c.tn == 4)
        return launch_large_m<4, 4, 4>(a);
    if (c.tm == 4 && c.tn == 2)
        return launch_large_m<4, 4, 2>(a);
    if (c.tm == 2 && c.tn == 2)
        return launch_large_m<4, 2, 2>(a);
    return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: no large-M kernel for tile %d,%d", c.tm, c.tn);
}
