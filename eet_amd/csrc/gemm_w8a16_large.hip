// Large-M fused dequant-GEMM (M > 32 apart from the 32-row-slab case; prefill;
// fp16-MFMA bound).
//
// Replaces the tensor-core side of fastertransformer::gemm_fp16_int_bias_act<uint8_t>
// (3rdparty/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm_template.h:48-177).
//
// A workgroup of WNW wavefronts side by side owns a block tile of TM*16 rows x
// WNW*TN*16 channels; each wavefront owns TM x TN tiles of
// v_mfma_f32_16x16x32_f16 (TM*TN*4 fp32 accumulator registers).  What bounds
// such a kernel on a CU is the LDS port (256 B/clk at best) against the matrix cores
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
// numbered so that the ones resident on an XCD at one time (workgroup i lands on
// XCD i % 8) cover a compact block of rows x columns and share both operands in its L2.
//
// A stage holds TM / 2 blocks of 4 KiB, one per pair of m-tiles (2u, 2u + 1):
// 16 "super-rows" of 256 B, super-row j holding row j of both m-tiles.  The MFMA
// operand of lane (g, j) for m-tile 2u + e, k half h -- the 16-byte piece 2g + h
// of row j -- sits at slot (4 * (2e + h) + g) ^ j of super-row j.  With that
// placement a ds_read_b128 of the whole wavefront runs at the full 256 B/clk of
// the LDS (measured: 128-byte rows with any XOR of the row index reach 150 B/clk).
// One DMA instruction fills 1 KiB = four super-rows; its lanes fetch whole
// 128-byte lines of eight activation rows (the XOR only permutes the lanes
// within a line).
#include "gemm_common.h"
#include "tuning.h"

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
    static_assert(TM % 2 == 0, "a stage block holds a pair of m-tiles");
    static_assert(kDmaStages * kStageVec * 16 <= 65536, "the stage ring must fit 64 KiB");
};

template <int WNW, int TM, int TN>
__global__ __launch_bounds__(64 * WNW) __attribute__((amdgpu_waves_per_eu(2))) void w8a16_large_m_kernel(
    const _Float16 *__restrict__ A, const u32x4 *__restrict__ Wp, const _Float16 *__restrict__ scale,
    _Float16 *__restrict__ C, int M, int N, int K, int m_blocks, int n_blocks,
    const _Float16 *__restrict__ residual, int epi, int ksplit, float *__restrict__ partial)
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
    // With ksplit > 1 (grid.y) the workgroup covers k-tiles [kbeg, kbeg + nk) only and
    // leaves its raw fp32 sums in partial[split][M][N] for the reduce kernel.
    const int split = blockIdx.y;
    const int kbeg = (int)((long)split * ktiles / ksplit);
    const int nk = (int)((long)(split + 1) * ktiles / ksplit) - kbeg;

    const int total = m_blocks * n_blocks;
    const int per_xcd = (total + 7) / 8;
    const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (tile >= total)
        return;
    // Tile order: bands of kBand column blocks across all row blocks, the column block running fastest inside a
    // band.  An XCD works through a contiguous range of that order, so the ~64 workgroups resident on it at one
    // time cover about 8 row blocks x 8 column blocks and every activation and weight line they fetch is shared
    // by eight of them in its L2 (with one column block after the other, 64 row blocks shared one weight block
    // and each fetched activation rows of its own from the fabric: M = 8192, 4096 -> 12288 went from 1.18 to
    // 1.28 PFLOP/s with the bands, the M = 2048 shapes gained 0-3 %).
    constexpr int kBand = 8;
    const int band = tile / (kBand * m_blocks), r = tile % (kBand * m_blocks);
    const int bw = min(kBand, n_blocks - band * kBand);   // column blocks of this band (the last one may be narrower)
    const int n_blk = band * kBand + r % bw, m_blk = r / bw;
    const int m0 = m_blk * S::kBM;
    const int nt0 = n_blk * (WNW * TN) + wave * TN;

    // Both operands are addressed through buffer resources: a 32-bit lane offset
    // plus a scalar offset per tile.  The range check of a buffer load covers the
    // lane offset only, not the scalar one: activation rows >= M are out of range
    // by their lane offset and read as zeros; the weight tile index lives in the
    // scalar offset, so an n-tile >= N/16 of a block that overhangs N is clamped
    // to the last real tile (its products are never stored).
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
        wtile[t] = (unsigned)min(nt0 + t, ntiles - 1) * (unsigned)ktiles * 1024u;

    // DMA instruction rg = wave * kPerWave + i fills slots [64 rg, 64 rg + 64): block u = rg / 4,
    // super-rows 4 (rg % 4) .. + 3.  Lane l writes slot s = l % 16 of super-row sj = 4 (rg % 4) + l / 16,
    // which holds piece 2 pg + h of row sj of m-tile 2u + e, where 4 (2e + h) + pg = s ^ sj.
    int aoff[S::kPerWave];
#pragma unroll
    for (int i = 0; i < S::kPerWave; ++i) {
        const int rg = wave * S::kPerWave + i, u = rg >> 2, sj = 4 * (rg & 3) + (lane >> 4);
        const int p = (lane & 15) ^ sj, pg = p & 3, h = (p >> 2) & 1, e = p >> 3;
        aoff[i] = ((2 * u + e) * 16 + sj) * K * 2 + (2 * pg + h) * 16;
    }
    int rs[4];  // operand slot of this lane within a block, by 2e + h
#pragma unroll
    for (int c = 0; c < 4; ++c)
        rs[c] = j * 16 + ((4 * c + g) ^ j);

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
        dma_tile(ahead, kbeg + min(kt + kDmaAhead, nk - 1));
        __builtin_amdgcn_sched_barrier(0);
        half8 w0[TN], w1[TN];
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            w0[t] = widen8(wb[t].x, wb[t].y);
            w1[t] = widen8(wb[t].z, wb[t].w);
        }
        __builtin_amdgcn_sched_barrier(0);
        load_w(wb, kbeg + min(kt + 2, nk - 1));
        half8 aop[2][2];
        aop[0][0] = __builtin_bit_cast(half8, cur[rs[0]]);
        aop[0][1] = __builtin_bit_cast(half8, cur[rs[1]]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) {
            if (mt + 1 < TM) {
                aop[(mt + 1) & 1][0] = __builtin_bit_cast(half8, cur[((mt + 1) >> 1) * 256 + rs[2 * ((mt + 1) & 1)]]);
                aop[(mt + 1) & 1][1] = __builtin_bit_cast(half8, cur[((mt + 1) >> 1) * 256 + rs[2 * ((mt + 1) & 1) + 1]]);
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
        // The DMA of tile kt+1 (issued two steps ago) must have landed before any wavefront reads it.  Accesses that
        // touch memory complete in the order issued, register loads and copies into LDS alike; one whose lanes are ALL
        // out of range (the row groups past M of a ragged block) completes at once, ahead of older copies (measured:
        // a counted wait over such accesses let an older copy through).  So the count has to hold with every such
        // access already gone.  Younger than that DMA are, among others, three weight batches (3 TN loads that always
        // touch memory); once no more than kPerWave + TN accesses are outstanding (the ones this step issued), the
        // complete ones include everything but the youngest kPerWave + TN <= 3 TN real ones, hence the DMA in
        // question.  Costs under 0.5 % against allowing the loads of two steps to be outstanding, which only timing
        // made safe on ragged blocks.
        // (A plain __syncthreads() would drain every outstanding load here: its
        // release fence waits for all DMA writes, including the ones just issued.)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(S::kPerWave + TN) : "memory");
    };

    // prologue: tiles 0..2 into stages 0..2, weights of tiles 0 and 1
    load_w(wraw[0], kbeg);
    dma_tile(st0, kbeg);
    load_w(wraw[1], kbeg + min(1, nk - 1));
    dma_tile(st1, kbeg + min(1, nk - 1));
    dma_tile(st2, kbeg + min(2, nk - 1));
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();

    int kt = 0;
    for (; kt + 4 <= nk; kt += 4) {
        step(st0, st3, wraw[0], kt);
        step(st1, st0, wraw[1], kt + 1);
        step(st2, st1, wraw[0], kt + 2);
        step(st3, st2, wraw[1], kt + 3);
    }
    if (kt < nk)
        step(st0, st3, wraw[0], kt);
    if (kt + 1 < nk)
        step(st1, st0, wraw[1], kt + 1);
    if (kt + 2 < nk)
        step(st2, st1, wraw[0], kt + 2);

    // acc[t][mt][r] of lane (g, j): row m0 + 16*mt + j, channel 16*(nt0+t) + 4*g + r
    const int mrow0 = m0 + j;
    if (ksplit > 1) {
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            if (nt0 + t >= ntiles)
                continue;
#pragma unroll
            for (int mt = 0; mt < TM; ++mt) {
                const int m = mrow0 + 16 * mt;
                if (m < M)
                    *reinterpret_cast<floatx4 *>(partial + ((size_t)split * M + m) * N + (nt0 + t) * 16 + 4 * g) =
                        acc[t][mt];
            }
        }
        return;
    }
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

// Second pass of a split-k launch: sums the ksplit partial results of 4 adjacent
// channels of one row, applies the per-channel scale and the epilogue, rounds once
// (gate and up are rounded to fp16 before SwiGLU, as the single-pass kernel does).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial,
                                                            const _Float16 *__restrict__ scale,
                                                            _Float16 *__restrict__ C,
                                                            const _Float16 *__restrict__ residual, int M, int N,
                                                            int ksplit, int epi)
{
    const int n_out = (epi == kEpiSwiglu) ? N / 2 : N;
    const int groups = n_out / 4;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * groups)
        return;
    const int m = idx / groups, o4 = (idx % groups) * 4;
    auto sum4 = [&](int n) {
        floatx4 s = *reinterpret_cast<const floatx4 *>(partial + (size_t)m * N + n);
        for (int k = 1; k < ksplit; ++k)
            s += *reinterpret_cast<const floatx4 *>(partial + ((size_t)k * M + m) * N + n);
        return s;
    };
    half4 o;
    if (epi == kEpiSwiglu) {
        const int ng = (o4 / 16) * 32 + o4 % 16, nu = ng + 16;  // gate tile 2u, up tile 2u+1
        const floatx4 sg = sum4(ng), su = sum4(nu);
        const half4 cg = *reinterpret_cast<const half4 *>(scale + ng), cu = *reinterpret_cast<const half4 *>(scale + nu);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float gate = (float)(_Float16)(sg[r] * (float)cg[r]);
            const float up = (float)(_Float16)(su[r] * (float)cu[r]);
            o[r] = (_Float16)(up * gate / (1.0f + __expf(-gate)));
        }
    } else {
        const floatx4 sv = sum4(o4);
        const half4 sc = *reinterpret_cast<const half4 *>(scale + o4);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            o[r] = (_Float16)(sv[r] * (float)sc[r]);
        if (epi == kEpiResidual)
            o = o + *reinterpret_cast<const half4 *>(residual + (size_t)m * N + o4);
    }
    *reinterpret_cast<half4 *>(C + (size_t)m * n_out + o4) = o;
}

template <int WNW, int TM, int TN>
int launch_large_m(const GemmArgs &a, int ksplit)
{
    using S = DmaShape<WNW, TM, TN>;
    const int m_blocks = (a.M + S::kBM - 1) / S::kBM, n_blocks = (a.N + S::kBN - 1) / S::kBN;
    const int grid = ((m_blocks * n_blocks + 7) / 8) * 8;
    float *partial = ksplit > 1 ? static_cast<float *>(a.ws) : nullptr;
    hipLaunchKernelGGL((w8a16_large_m_kernel<WNW, TM, TN>), dim3(grid, ksplit), dim3(S::kThreads), 0, a.st, a.A, a.Wp,
                       a.scale, a.C, a.M, a.N, a.K, m_blocks, n_blocks, a.residual, a.epi, ksplit, partial);
    EET_HIP_CHECK(hipGetLastError());
    if (ksplit > 1) {
        const int items = a.M * ((a.epi == kEpiSwiglu ? a.N / 2 : a.N) / 4);
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((items + 255) / 256), dim3(256), 0, a.st, partial, a.scale, a.C,
                           a.residual, a.M, a.N, ksplit, a.epi);
        EET_HIP_CHECK(hipGetLastError());
    }
    return EET_OK;
}

struct LargeMConfig {
    int tm, tn;  // m-tiles and n-tiles of 16 per wavefront; the block is tm*16 rows x 4*tn*16 channels
    int ksplit;  // > 1: that many workgroups share a tile's k range (needs the fp32 workspace)
};

// Shape -> tile.  Measured on MI355X (M = 33 .. 8192, LLaMA-7B and Baichuan-13B shapes):
//   128 x 256 (two workgroups per CU) is the fastest tile once it yields a few
//     hundred workgroups;
//   64 x 320 wins when it divides the problem into whole rounds of 512 workgroups
//     where 128 x 256 leaves a CU with two tiles against one elsewhere (M = 2048,
//     N = 5120: 512 tiles, two per CU, instead of 320);
//   64 x 256, 64 x 128 and 32 x 128 keep the chip occupied for M in the tens and
//     hundreds, where the k-loop latency of a few large tiles would dominate.
// Estimated time (us) of tile (tm, tn) with the k range split ks ways, for launches
// too small to fill the chip.  Fitted to MI355X measurements (M = 40 .. 512, LLaMA-7B
// shapes, within ~10 %): a workgroup alone on its CU needs `lat` us per k-tile
// (load -> widen -> MFMA latency chain), co-resident workgroups share the CU's
// L2 bandwidth at `thr` us per k-tile each; a split launch pays a second kernel
// (~2 us) that reads what the first wrote (ks * M * N fp32, ~4 TB/s effective).
struct SplitTile {
    int tm, tn;
    double lat, thr;
};
constexpr SplitTile kSplitTiles[2] = {{2, 2, 0.26, 0.14}, {4, 2, 0.33, 0.23}};

double split_cost_us(int M, int N, int K, const SplitTile &t, int ks)
{
    const int wgs = ((M + t.tm * 16 - 1) / (t.tm * 16)) * ((N + t.tn * 64 - 1) / (t.tn * 64)) * ks;
    const double load = wgs <= 512 ? (double)((wgs + 255) / 256) : wgs / 256.0;
    const double per_tile = t.lat > t.thr * load ? t.lat : t.thr * load;
    double us = 2.5 + (K / 64.0 / ks) * per_tile;
    if (ks > 1)
        us += 2.0 + (double)ks * M * N * 8.0 / 4e6;
    return us;
}

LargeMConfig pick_large_m(int M, int N, int K, int epi, bool may_split)
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
                return LargeMConfig{4, 5, 1};
        }
        return LargeMConfig{8, 4, 1};
    }
    if (wgs(64, 256) >= 600)
        return LargeMConfig{4, 4, 1};
    // Fewer tiles than fill the chip twice: 32 x 128 or 64 x 128, and the k range of
    // a tile may be shared by up to 8 workgroups (at least 8 k-tiles each) whose fp32
    // partial sums a small second kernel adds.
    const int ktiles = K / 64;
    LargeMConfig best{2, 2, 1};
    double best_us = 1e30;
    for (const SplitTile &t : kSplitTiles)
        for (int ks = 1; ks <= (may_split ? 8 : 1); ++ks) {
            if (ks > 1 && ktiles / ks < 8)
                break;
            const double us = split_cost_us(M, N, K, t, ks);
            if (us < best_us) {
                best_us = us;
                best = LargeMConfig{t.tm, t.tn, ks};
            }
        }
    return best;
}

}  // namespace

size_t eet::large_m_workspace(int M, int N, int K, int epi)
{
    const LargeMConfig c = pick_large_m(M, N, K, epi, true);
    return c.ksplit > 1 ? (size_t)c.ksplit * M * N * sizeof(float) : 0;
}

int eet::run_large_m(const GemmArgs &a)
{
    // the kernel addresses A rows and the packed weights with 32-bit byte offsets
    if ((size_t)a.K * a.N >= (1ull << 31) || (size_t)a.K * 2 * 256 >= (1ull << 31))
        return eet::fail(EET_ERR_UNSUPPORTED_SHAPE, "eet_gemm_w8a16: K x N = %d x %d exceeds the 2 GiB weight limit",
                         a.K, a.N);
    // the split needs room for ksplit x M x N fp32; without it the best single-pass tile
    auto fits = [&](int ks) {
        return ks <= 1 || (a.ws != nullptr && reinterpret_cast<uintptr_t>(a.ws) % 16 == 0 &&
                           a.ws_bytes >= (size_t)ks * a.M * a.N * sizeof(float));
    };
    LargeMConfig c = pick_large_m(a.M, a.N, a.K, a.epi, true);
    if (!fits(c.ksplit))
        c = pick_large_m(a.M, a.N, a.K, a.epi, false);
    const eet::Tuning &tune = eet::tuning();
    if (tune.has_large_m) {  // "tm,tn[,ksplit]": runs when such a tile exists, else the table's choice stands
        const int tm = tune.large_m_tm, tn = tune.large_m_tn;
        const bool exists = (tm == 8 && tn == 4) || (tm == 4 && (tn == 5 || tn == 4 || tn == 2)) || (tm == 2 && tn == 2);
        if (exists && (a.epi != kEpiSwiglu || tn % 2 == 0))
            c = LargeMConfig{tm, tn, tune.large_m_ksplit > 0 ? tune.large_m_ksplit : 1};
        if (!fits(c.ksplit))
            c.ksplit = 1;
    }
    if (c.ksplit < 1 || c.ksplit > a.K / 64)
        c.ksplit = 1;
    if (c.tm == 8 && c.tn == 4)
        return launch_large_m<4, 8, 4>(a, c.ksplit);
    if (c.tm == 4 && c.tn == 5)
        return launch_large_m<4, 4, 5>(a, c.ksplit);
    if (c.tm == 4 && c.tn == 4)
        return launch_large_m<4, 4, 4>(a, c.ksplit);
    if (c.tm == 4 && c.tn == 2)
        return launch_large_m<4, 4, 2>(a, c.ksplit);
    if (c.tm == 2 && c.tn == 2)
        return launch_large_m<4, 2, 2>(a, c.ksplit);
    return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_gemm_w8a16: no large-M kernel for tile %d,%d", c.tm, c.tn);
}
