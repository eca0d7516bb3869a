// Fused dequant-GEMM: C[M][N] = A[M][K] (fp16) . (int8 W[K][N] * scale[N]).
//
// Replaces fastertransformer::gemm_fp16_int_bias_act<uint8_t>
// (3rdparty/cutlass_kernels/fpA_intB_gemm.cu:35-62) as EET calls it: no bias,
// no activation (csrc/op/llama_mmha.cpp:313-337).  EET never passes the split-k
// workspace; here it is optional and used for M in the tens to hundreds.
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
//
// Built a second time with -DEET_TIMELINE into the bench-only library: the same kernels with five
// clock readings per workgroup (entry, first batch multiplied, k loop done, stores issued, stores
// acknowledged), under entry-point names of their own, so that the measurement harness can say where the
// time of a launch goes.  Nothing of it is compiled into the operator library.
#if defined(EET_TIMELINE)
#define eet_gemm_w8a16 eet_timeline_gemm_w8a16
#define eet_gemm_w8a16_fused eet_timeline_gemm_w8a16_fused
#define eet_gemm_w8a16_chained eet_timeline_gemm_w8a16_chained
#define eet_gemm_w8a16_small_m_shape eet_timeline_gemm_w8a16_small_m_shape
#define eet_gemm_w8a16_workspace eet_timeline_gemm_w8a16_workspace
#endif
#include <hip/hip_runtime.h>

#include <hip/hip_ext.h>

#include "chain.h"
#include "gemm_common.h"
#include "tuning.h"

using namespace eet;

#if defined(EET_TIMELINE)
#define EET_TL_PARAM , unsigned long long *tl
#define EET_TL_ARG , timeline_next(grid_of_launch)
#define EET_TL_NONE , nullptr
#define EET_TL_STAMP(i)                                      \
    do {                                                     \
        if (tl != nullptr && threadIdx.x == 0)               \
            tl_t[i] = wall_clock64();                        \
    } while (0)
namespace {
constexpr int kTlStamps = 24, kTlMaxWgs = 1024;   // 8 readings of the workgroup, then one per wavefront
unsigned long long *g_tl_buf = nullptr;   // [launch][kTlMaxWgs][kTlStamps], device memory
int g_tl_cap = 0, g_tl_n = 0;
int g_tl_grid[4096];
unsigned long long *timeline_next(int workgroups)
{
    if (g_tl_buf == nullptr || g_tl_n >= g_tl_cap || g_tl_n >= 4096 || workgroups > kTlMaxWgs)
        return nullptr;
    g_tl_grid[g_tl_n] = workgroups;
    return g_tl_buf + (size_t)(g_tl_n++) * kTlMaxWgs * kTlStamps;
}
}  // namespace
#else
#define EET_TL_PARAM
#define EET_TL_ARG
#define EET_TL_NONE
#define EET_TL_STAMP(i) do { } while (0)
#endif

namespace {

// One batch of U k-tiles as it comes back from memory: the raw weight tiles of
// NT n-tiles, and the activations of RG groups of 8 rows, loaded row-wise.
template <int NT, int RG, int U>
struct Batch {
    u32x4 w[U][NT];
    u32x4 a[U][RG];
    u32x4 gam[U];  // RMSnorm weights of the lane's piece (only with the RMSnorm prologue)
};

// Activation loads are issued so that a wavefront reads whole 128-byte lines:
// lane l fetches the 16-byte piece l%8 of row 8*r + l/8 of the k-tile (8 rows
// x 128 B = 1 KiB per instruction).  Letting each lane fetch its own MFMA
// operand straight from the row-major matrix instead costs 16 half-used lines
// per instruction and measured 1.4 us (M = 8) to 2.5 us (M = 16) on a 4 us
// kernel.
//
// The weights come through a buffer resource over the whole packed matrix: the
// n-tile and k-tile select a wavefront-uniform (scalar) offset, the lane adds
// 16 * lane.  With `valid` false (the request one batch past the end, which the
// main loop issues without a branch so that its waits stay exact) the lane
// offset is moved out of range: zeros come back and no memory is touched; the
// activations then re-read k-tile 0.
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
template <int NT, int RG, int WAVES, int U, bool RMS>
__device__ __forceinline__ void load_batch(Batch<NT, RG, U> &b, __amdgpu_buffer_rsrc_t wrsrc,
                                           const unsigned (&wtile)[NT], int lane, const u32x4 *const (&abase)[RG],
                                           const u32x4 *gbase, int kt, bool valid)
{
    constexpr int kStream = 2;  // aux bits: non-temporal (every weight is read exactly once)
    const unsigned voff = valid ? (unsigned)lane * 16u : 0x80000000u;
    // All weight loads (HBM latency) go out first, then the activation loads
    // (L2 hits); loads return in issue order.
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            b.w[u][t] = __builtin_bit_cast(
                u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, voff, wtile[t] + (unsigned)(kt + u * WAVES) * 1024u,
                                                             kStream));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < RG; ++r)
            b.a[u][r] = abase[r][valid ? (kt + u * WAVES) * 8 : 0];
    if (RMS) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            b.gam[u] = gbase[valid ? (kt + u * WAVES) * 8 : 0];
    }
    __builtin_amdgcn_sched_barrier(0);
}
#endif

// The two halves of load_batch on their own, for the chained kernel: its first weight
// batches are requested before the wait for the producer, the activations after it.  The
// activations go through a buffer resource with the sc1 bit (agent scope: served by the L2,
// which the hardware keeps coherent across XCDs for such accesses, and never by a stale L1
// line); a request that is not `valid` is moved out of range.
#if defined(__HIP_DEVICE_COMPILE__)
constexpr int kAgentScope = 16;   // aux bits of a buffer access: sc1
template <int NT, int RG, int WAVES, int U>
__device__ __forceinline__ void load_batch_w(Batch<NT, RG, U> &b, __amdgpu_buffer_rsrc_t wrsrc,
                                             const unsigned (&wtile)[NT], int lane, int kt, bool valid)
{
    constexpr int kStream = 2;
    const unsigned voff = valid ? (unsigned)lane * 16u : 0x80000000u;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            b.w[u][t] = __builtin_bit_cast(
                u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, voff, wtile[t] + (unsigned)(kt + u * WAVES) * 1024u,
                                                             kStream));
    __builtin_amdgcn_sched_barrier(0);
}

template <int NT, int RG, int WAVES, int U, bool RMS>
__device__ __forceinline__ void load_batch_a_chained(Batch<NT, RG, U> &b, __amdgpu_buffer_rsrc_t arsrc,
                                                     const unsigned (&aoff)[RG], const u32x4 *gbase, int kt, bool valid)
{
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < RG; ++r)
            b.a[u][r] = __builtin_bit_cast(
                u32x4, __builtin_amdgcn_raw_buffer_load_b128(arsrc, valid ? aoff[r] : 0x80000000u,
                                                             (unsigned)(kt + u * WAVES) * 128u, kAgentScope));
    if (RMS) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            b.gam[u] = gbase[valid ? (kt + u * WAVES) * 8 : 0];
    }
    __builtin_amdgcn_sched_barrier(0);
}
#endif

// The row-wise activation pieces are turned into MFMA operands through a
// wavefront-private LDS slab: lane (g, j) of operand half h needs piece
// 2*g + h of row j.  Piece p of row jr is kept at slot jr*8 + (p ^ jr), which
// makes both the 16-byte writes and the 16-byte reads bank-conflict free.
template <int NT, int RG, int U, bool RMS>
__device__ __forceinline__ void mma_batch(const Batch<NT, RG, U> &b, floatx4 (&acc)[NT][(RG + 1) / 2],
                                          u32x4 *slab, int lane, float (&ss)[RG])
{
    constexpr int MT = (RG + 1) / 2;
    const int g = lane >> 4, j = lane & 15;
    const int wslot = (lane & ~7) | ((lane & 7) ^ (lane >> 3));
    const int jr = j & 7;
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int r = 0; r < RG; ++r) {
            u32x4 piece = b.a[u][r];
            if (RMS) {
                // RMSnorm prologue: accumulate sum(x^2) of the row and feed x * gamma
                // (fp16) to the MFMA; 1/rms is applied to the fp32 sum in the epilogue.
                const half8 x = __builtin_bit_cast(half8, piece);
                const half2v x0 = __builtin_shufflevector(x, x, 0, 1), x1 = __builtin_shufflevector(x, x, 2, 3);
                const half2v x2 = __builtin_shufflevector(x, x, 4, 5), x3 = __builtin_shufflevector(x, x, 6, 7);
                ss[r] = __builtin_amdgcn_fdot2(x0, x0, ss[r], false);
                ss[r] = __builtin_amdgcn_fdot2(x1, x1, ss[r], false);
                ss[r] = __builtin_amdgcn_fdot2(x2, x2, ss[r], false);
                ss[r] = __builtin_amdgcn_fdot2(x3, x3, ss[r], false);
                piece = __builtin_bit_cast(u32x4, x * __builtin_bit_cast(half8, b.gam[u]));
            }
            slab[(u * RG + r) * 64 + wslot] = piece;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        half8 op[MT][2];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            // rows 16*mt + j; a row group that was not loaded (M <= 8 with one
            // group) is replaced by group 0: those columns are never written
            const int r = (2 * mt + (j >> 3) < RG) ? 2 * mt + (j >> 3) : 0;
#pragma unroll
            for (int h = 0; h < 2; ++h)
                op[mt][h] = __builtin_bit_cast(half8, slab[(u * RG + r) * 64 + jr * 8 + ((2 * g + h) ^ jr)]);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const half8 w0 = widen8(b.w[u][t].x, b.w[u][t].y);
            const half8 w1 = widen8(b.w[u][t].z, b.w[u][t].w);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, op[mt][0], acc[t][mt], 0, 0, 0);
                acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, op[mt][1], acc[t][mt], 0, 0, 0);
            }
        }
    }
}

// NT: n-tiles per workgroup.  RG: groups of 8 activation rows (M <= 8 * RG).
// RMS: RMSnorm prologue compiled in (it costs ~20-30 registers, so the plain
// GEMM is a separate instantiation).  CHAIN: the chained form (chain.h): the first two
// weight batches are requested, then the workgroup waits for the producer of A and of the
// residual rows, reads both with agent-scope loads, writes C with agent-scope stores and
// signals its own completion; `link` is ignored otherwise.
//
// MODE kPair2 / kPair4: the k range of a group of NT n-tiles is shared by KS = 2 or 4 workgroups
// (grid.y = KS), so that a launch whose N leaves one n-tile per CU can give a workgroup NT = KS (or
// more) n-tiles and still fill the chip: every workgroup reads all M x K / KS activations of its k
// share, i.e. the L2 -> CU activation traffic of the launch falls by the factor NT.  Each workgroup
// writes its fp32 tile sums to its slot of `pair.sums` (agent-scope stores), then takes a ticket from
// the group's counter; the one that arrives LAST adds the others' sums to its own and finishes the
// tiles (scale, epilogue, store) and puts the counter back to zero.  Nobody waits for anybody.  Slots and
// counters live in the CALLER's workspace (so calls on different streams never share them): the
// counters must be zero before the first launch that uses a workspace; every launch leaves them zero.
struct PairArgs {
    floatx4 *sums;      // [groups][KS][NT * MT][64]
    unsigned *tickets;  // [groups], 64 bytes apart
};
constexpr int kPlain = 0, kChained = 1, kPair2 = 2, kPair4 = 4;
constexpr int kPairTiles = 10;   // NT * MT <= 10 tiles per group

template <int NT, int RG, int WAVES, int U, bool RMS, int MODE>
__global__ __launch_bounds__(WAVES * 64) void w8a16_small_m_kernel(
    // argument order: the first 14 dwords are in SGPRs when a wavefront starts (kernel-argument preload); they
    // hold what the first requests of the wavefront need, the rest is fetched while those are in flight
    const _Float16 *__restrict__ A, const u32x4 *__restrict__ Wp, int M, int N, int K, int epi,
    const _Float16 *__restrict__ residual, const _Float16 *__restrict__ rms_gamma,
    const _Float16 *__restrict__ scale, _Float16 *__restrict__ C, float rms_eps, eet::ChainLink link,
    PairArgs pair EET_TL_PARAM)
{
    constexpr bool CHAIN = MODE == kChained, PAIR = MODE == kPair2 || MODE == kPair4;
    constexpr int KS = PAIR ? MODE : 1;
    static_assert(!PAIR || (!RMS && NT * ((RG + 1) / 2) <= kPairTiles), "k split: no RMSnorm prologue, at most 10 tiles");
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    constexpr int MT = (RG + 1) / 2;
#if defined(EET_TIMELINE)
    unsigned long long tl_t[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    __shared__ unsigned long long tl_wave_end[WAVES];
    __shared__ unsigned tl_wave_hw[WAVES];
    auto tl_flush = [&]() {
        if (tl != nullptr && threadIdx.x == 0) {
            unsigned long long *q = tl + (size_t)(blockIdx.y * gridDim.x + blockIdx.x) * kTlStamps;
            for (int i = 0; i < 8; ++i)
                q[i] = tl_t[i];
        }
    };
#endif
    EET_TL_STAMP(0);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: feeds scalar offsets
    const int g = lane >> 4, j = lane & 15;
    const int ktiles = K >> 6;
    const int ntiles = N >> 4;
    const int nt0 = blockIdx.x * NT;

    // LDS: first the per-wavefront activation slabs, later (after a barrier)
    // the partial sums of the cross-wavefront reduction.
    constexpr int kSlabVec = U * RG * 64;                      // u32x4 per wavefront
    constexpr int kStageBytes = WAVES * kSlabVec * 16;
    constexpr int kRedBytes = WAVES * NT * MT * 64 * 16;
    // The two regions share memory only when both together would not fit 64 KiB
    // (sharing costs a second barrier in the epilogue).
    constexpr bool kAlias = kStageBytes + kRedBytes > 65536;
    constexpr int kLdsBytes = kAlias ? (kStageBytes > kRedBytes ? kStageBytes : kRedBytes) : kStageBytes + kRedBytes;
    __shared__ __attribute__((aligned(16))) unsigned char lds[kLdsBytes];
    u32x4 *slab = reinterpret_cast<u32x4 *>(lds) + wave * kSlabVec;

    floatx4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // A tile index past the end is clamped: its results are never written.
    const __amdgpu_buffer_rsrc_t wrsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<u32x4 *>(Wp), 0, (unsigned)((size_t)K * N), 0x00020000);
    unsigned wtile[NT];  // byte offset of the n-tile's first k-tile
#pragma unroll
    for (int t = 0; t < NT; ++t)
        wtile[t] = (unsigned)min(nt0 + t, ntiles - 1) * (unsigned)ktiles * 1024u;
    // Rows past M read row M-1: column m of the product depends only on
    // activation row m, and rows >= M are not written.
    const u32x4 *abase[RG];
#pragma unroll
    for (int r = 0; r < RG; ++r) {
        int m = min(8 * r + (lane >> 3), M - 1);
        abase[r] = reinterpret_cast<const u32x4 *>(A + (size_t)m * K) + (lane & 7);
    }

    // Epilogue operands (per-channel scales, residual rows) are requested first
    // of all, so that a miss in L2 is long over when the epilogue needs them.
    // An output unit is
    // one (n-tile, m-tile) product, or for the SwiGLU epilogue the pair of
    // adjacent n-tiles (gate, up) of one m-tile.
    constexpr int kMaxUnits = (NT * MT + WAVES - 1) / WAVES;
    const int units = (epi == kEpiSwiglu) ? (NT / 2) * MT : NT * MT;
    half4 sc0[kMaxUnits], sc1[kMaxUnits], res[kMaxUnits];
    {
        // The residual rows come through a buffer resource that is empty unless the epilogue adds them: the
        // load needs no branch then (behind a branch the compiler merges the loaded registers right after it,
        // i.e. makes the wavefront wait a whole memory latency before its first weight request).
        [[maybe_unused]] const __amdgpu_buffer_rsrc_t res_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<_Float16 *>(residual), 0, (!CHAIN && epi == kEpiResidual) ? (unsigned)M * (unsigned)N * 2u : 0u,
            0x00020000);
        int idx = 0;
        for (int unit = wave; unit < units; unit += WAVES, ++idx) {
            const int mt = unit % MT;
            const int t = (epi == kEpiSwiglu) ? 2 * (unit / MT) : unit / MT;
            const int nt = min(nt0 + t, ntiles - 1);
            sc0[idx] = *reinterpret_cast<const half4 *>(scale + nt * 16 + 4 * g);
            if (epi == kEpiSwiglu)
                sc1[idx] = *reinterpret_cast<const half4 *>(scale + min(nt + 1, ntiles - 1) * 16 + 4 * g);
            if constexpr (!CHAIN) {
                const int m = min(mt * 16 + j, M - 1);
                res[idx] = __builtin_bit_cast(
                    half4, __builtin_amdgcn_raw_buffer_load_b64(
                               res_rsrc, ((unsigned)m * (unsigned)N + (unsigned)(nt * 16 + 4 * g)) * 2u, 0, 0));
            }
        }
    }

    __builtin_amdgcn_sched_barrier(0);

    constexpr bool rms = RMS;
    const u32x4 *gbase = rms ? reinterpret_cast<const u32x4 *>(rms_gamma) + (lane & 7) : nullptr;
    float ss[RG];
#pragma unroll
    for (int r = 0; r < RG; ++r)
        ss[r] = 0.f;

    // This wavefront's k-tiles are wave, wave + WAVES, ...; they are taken in
    // batches of U with the next batch's loads in flight while the current one
    // is multiplied (two register buffers).  The request for the batch after
    // next is issued on every pass, past the end too (where it costs nothing):
    // with a branch around it the compiler has to wait for that request as well
    // before the second multiply, i.e. it empties the pipeline once per pass.
    // this workgroup's k-tiles: all of them, or with the k split the share blockIdx.y names
    const int kt_begin = PAIR ? (int)((long)blockIdx.y * ktiles / KS) : 0;
    const int kt_end = PAIR ? (int)((long)(blockIdx.y + 1) * ktiles / KS) : ktiles;
    const int span = kt_end - kt_begin;
    const int mine = span > wave ? (span - wave + WAVES - 1) / WAVES : 0;
    const int nbatch = mine / U;
    constexpr int STEP = U * WAVES;
    int kt = kt_begin + wave;
    if constexpr (CHAIN) {
        // Chained form.  The weights of the first two batches depend on nothing and are requested
        // at once; then the wait for the producer; then the residual rows and the activations of
        // those two batches.  From there on a batch is multiplied and its buffer refilled with the
        // batch after next, so the wait before a multiply counts exactly the younger batch.
        const unsigned a_bytes = (unsigned)M * (unsigned)K * 2u;
        unsigned aoff[RG];
#pragma unroll
        for (int r = 0; r < RG; ++r)
            aoff[r] = ((unsigned)min(8 * r + (lane >> 3), M - 1) * (unsigned)K + (unsigned)(lane & 7) * 8u) * 2u;
        Batch<NT, RG, U> b0, b1;
        load_batch_w<NT, RG, WAVES, U>(b0, wrsrc, wtile, lane, kt, nbatch > 0);
        load_batch_w<NT, RG, WAVES, U>(b1, wrsrc, wtile, lane, kt + STEP, nbatch > 1);
        eet::chain_wait(link);
        // the compiler must not know that these are the kernel's read-only arguments: what they
        // point to has just been written by another kernel
        const _Float16 *A_now = A, *res_now = residual;
        asm volatile("" : "+s"(A_now), "+s"(res_now)::"memory");
        const __amdgpu_buffer_rsrc_t arsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(A_now), 0, a_bytes, 0x00020000);
        if (epi == kEpiResidual) {
            const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<_Float16 *>(res_now), 0, (unsigned)M * (unsigned)N * 2u, 0x00020000);
            int idx = 0;
            for (int unit = wave; unit < units; unit += WAVES, ++idx) {
                const int mt = unit % MT, t = unit / MT;
                const int nt = min(nt0 + t, ntiles - 1), m = min(mt * 16 + j, M - 1);
                const unsigned off = ((unsigned)m * (unsigned)N + (unsigned)(nt * 16 + 4 * g)) * 2u;
                res[idx] = __builtin_bit_cast(half4, __builtin_amdgcn_raw_buffer_load_b64(rrsrc, off, 0, kAgentScope));
            }
        }
        load_batch_a_chained<NT, RG, WAVES, U, RMS>(b0, arsrc, aoff, gbase, kt, nbatch > 0);
        load_batch_a_chained<NT, RG, WAVES, U, RMS>(b1, arsrc, aoff, gbase, kt + STEP, nbatch > 1);
        int i = 0;
        for (; i + 2 <= nbatch; i += 2) {
            mma_batch<NT, RG, U, RMS>(b0, acc, slab, lane, ss);
            load_batch_w<NT, RG, WAVES, U>(b0, wrsrc, wtile, lane, kt + 2 * STEP, i + 2 < nbatch);
            load_batch_a_chained<NT, RG, WAVES, U, RMS>(b0, arsrc, aoff, gbase, kt + 2 * STEP, i + 2 < nbatch);
            mma_batch<NT, RG, U, RMS>(b1, acc, slab, lane, ss);
            load_batch_w<NT, RG, WAVES, U>(b1, wrsrc, wtile, lane, kt + 3 * STEP, i + 3 < nbatch);
            load_batch_a_chained<NT, RG, WAVES, U, RMS>(b1, arsrc, aoff, gbase, kt + 3 * STEP, i + 3 < nbatch);
            kt += 2 * STEP;
        }
        if (i < nbatch) {
            mma_batch<NT, RG, U, RMS>(b0, acc, slab, lane, ss);
            kt += STEP;
        }
        for (; kt < kt_end; kt += WAVES) {
            Batch<NT, RG, 1> b;
            load_batch_w<NT, RG, WAVES, 1>(b, wrsrc, wtile, lane, kt, true);
            load_batch_a_chained<NT, RG, WAVES, 1, RMS>(b, arsrc, aoff, gbase, kt, true);
            mma_batch<NT, RG, 1, RMS>(b, acc, slab, lane, ss);
        }
    } else {
        {
            Batch<NT, RG, U> b0, b1;
            load_batch<NT, RG, WAVES, U, RMS>(b0, wrsrc, wtile, lane, abase, gbase, kt, nbatch > 0);
            int i = 0;
            for (; i + 2 <= nbatch; i += 2) {
                load_batch<NT, RG, WAVES, U, RMS>(b1, wrsrc, wtile, lane, abase, gbase, kt + STEP, true);
                mma_batch<NT, RG, U, RMS>(b0, acc, slab, lane, ss);
#if defined(EET_TIMELINE)
                if (i == 0)
                    EET_TL_STAMP(1);
#endif
                load_batch<NT, RG, WAVES, U, RMS>(b0, wrsrc, wtile, lane, abase, gbase, kt + 2 * STEP, i + 2 < nbatch);
                mma_batch<NT, RG, U, RMS>(b1, acc, slab, lane, ss);
                kt += 2 * STEP;
            }
            if (i < nbatch) {
                mma_batch<NT, RG, U, RMS>(b0, acc, slab, lane, ss);
                kt += STEP;
            }
        }
        for (; kt < kt_end; kt += WAVES) {
            Batch<NT, RG, 1> b;
            load_batch<NT, RG, WAVES, 1, RMS>(b, wrsrc, wtile, lane, abase, gbase, kt, true);
            mma_batch<NT, RG, 1, RMS>(b, acc, slab, lane, ss);
        }
    }

    EET_TL_STAMP(2);
#if defined(EET_TIMELINE)
    if (tl != nullptr && (threadIdx.x & 63) == 0) {
        tl_wave_end[threadIdx.x >> 6] = wall_clock64();   // every wavefront's end of the k loop
        tl_wave_hw[threadIdx.x >> 6] = __builtin_amdgcn_s_getreg(63492) & 0xffff;
    }
#endif
    // RMSnorm prologue: each wavefront's share of sum(x^2) per row.  Lanes
    // 8*q .. 8*q+7 hold pieces of row 8*r + q.
    __shared__ float rowss[WAVES][RG * 8];
    if (rms) {
#pragma unroll
        for (int r = 0; r < RG; ++r) {
            float v = ss[r];
            v += __shfl_xor(v, 1, 64);
            v += __shfl_xor(v, 2, 64);
            v += __shfl_xor(v, 4, 64);
            if ((lane & 7) == 0)
                rowss[wave][r * 8 + (lane >> 3)] = v;
        }
    }

    // Cross-wavefront reduction.  acc[t][mt][r] of lane (g, j) is the product
    // for channel 16*(nt0+t) + 4*g + r and row 16*mt + j.
    if (kAlias)
        __syncthreads();  // every wavefront is done with its activation slab
    floatx4 *red = reinterpret_cast<floatx4 *>(lds + (kAlias ? 0 : kStageBytes));  // [WAVES][NT * MT][64]
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            red[(wave * NT * MT + t * MT + mt) * 64 + lane] = acc[t][mt];
    __syncthreads();
#if defined(EET_TIMELINE)
    EET_TL_STAMP(5);   // all wavefronts have left the k loop and written their partial sums
    if (tl != nullptr && threadIdx.x == 0) {
        unsigned long long lo = ~0ull, sum = 0;
        for (int w = 0; w < WAVES; ++w) {
            lo = tl_wave_end[w] < lo ? tl_wave_end[w] : lo;
            sum += tl_wave_end[w] - tl_t[0];
        }
        tl_t[6] = lo;                    // the first wavefront to finish its k loop
        tl_t[7] = tl_t[0] + sum / WAVES; // the mean over the wavefronts
        // per wavefront: the end of its k loop after the workgroup's entry (low 32 bits) and where it ran
        // (HW_ID bits 0-15 above them: wave slot, SIMD, CU, shader array and engine)
        unsigned long long *q = tl + (size_t)(blockIdx.y * gridDim.x + blockIdx.x) * kTlStamps + 8;
        for (int w = 0; w < WAVES; ++w)
            q[w] = ((tl_wave_end[w] - tl_t[0]) & 0xffffffffull) | ((unsigned long long)tl_wave_hw[w] << 32);
    }
#endif
    auto tile_sum = [&](int tile) {
        floatx4 s = red[tile * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            s += red[(w * NT * MT + tile) * 64 + lane];
        return s;
    };
    // four output halves of one lane; the chained form stores them write-through (agent scope)
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc(
        C, 0, (unsigned)M * (unsigned)(epi == kEpiSwiglu ? N / 2 : N) * 2u, 0x00020000);
    auto store_out = [&](half4 o, size_t elem) {
        if constexpr (CHAIN)
            __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, o), crsrc, (unsigned)elem * 2u, 0, kAgentScope);
        else
            *reinterpret_cast<half4 *>(C + elem) = o;
    };
    // k split: publish this share's tile sums, take a ticket; all but the last arrival are done, the
    // last adds the others' sums and goes on to the epilogue.
    floatx4 whole[kMaxUnits];
    if constexpr (PAIR) {
        constexpr int kTiles = NT * MT;
        const __amdgpu_buffer_rsrc_t prs = __builtin_amdgcn_make_buffer_rsrc(
            pair.sums + ((size_t)blockIdx.x * KS * kTiles) * 64, 0, (unsigned)KS * kTiles * 64u * 16u, 0x00020000);
        int i2 = 0;
        for (int unit = wave; unit < units; unit += WAVES, ++i2) {
            whole[i2] = tile_sum(unit);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, whole[i2]), prs,
                                                   (unsigned)(((blockIdx.y * kTiles + unit) * 64 + lane) * 16), 0,
                                                   kAgentScope);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __shared__ unsigned ticket;
        __syncthreads();
        if (threadIdx.x == 0)
            ticket = __hip_atomic_fetch_add(pair.tickets + blockIdx.x * 16, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket != KS - 1) {
#if defined(EET_TIMELINE)
            EET_TL_STAMP(3);
            EET_TL_STAMP(4);
            tl_flush();
#endif
            return;   // the last arrival will find these sums and finish
        }
        if (threadIdx.x == 0)   // ready for the next launch on this workspace
            __hip_atomic_store(pair.tickets + blockIdx.x * 16, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // The shares are added in the order of the k range, whichever workgroup came last: the rounding of
        // the sum, and with it the result, does not depend on the order of arrival.
        i2 = 0;
        for (int unit = wave; unit < units; unit += WAVES, ++i2) {
            floatx4 part[KS];
#pragma unroll
            for (int o = 0; o < KS; ++o)
                part[o] = __builtin_bit_cast(
                    floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                                 prs, (unsigned)(((o * kTiles + unit) * 64 + lane) * 16), 0, kAgentScope));
            floatx4 tot = blockIdx.y == 0 ? whole[i2] : part[0];
#pragma unroll
            for (int o = 1; o < KS; ++o)
                tot += (int)blockIdx.y == o ? whole[i2] : part[o];
            whole[i2] = tot;
        }
    }
    int idx = 0;
    for (int unit = wave; unit < units; unit += WAVES, ++idx) {
        const int mt = unit % MT;
        const int m = mt * 16 + j;
        float inv = 1.0f;
        if (rms) {
            const int row = min(m, RG * 8 - 1);
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
                tot += rowss[w][row];
            inv = rsqrtf(tot / (float)K + rms_eps);
        }
        if (epi == kEpiSwiglu) {
            const int t = 2 * (unit / MT);
            const floatx4 sg = tile_sum(t * MT + mt), su = tile_sum((t + 1) * MT + mt);
            if (nt0 + t + 1 < ntiles && m < M) {
                // gate and up are rounded to fp16 first, as the separate GEMMs would leave them
                half4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float gate = (float)(_Float16)(sg[r] * (float)sc0[idx][r] * inv);
                    const float up = (float)(_Float16)(su[r] * (float)sc1[idx][r] * inv);
                    o[r] = (_Float16)(up * gate / (1.0f + __expf(-gate)));
                }
                const int n = ((nt0 + t) / 2) * 16 + 4 * g;
                store_out(o, (size_t)m * (N / 2) + n);
            }
        } else {
            const int t = unit / MT;
            const floatx4 s = PAIR ? whole[idx] : tile_sum(unit);
            if (nt0 + t < ntiles && m < M) {
                const int n = (nt0 + t) * 16 + 4 * g;
                half4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    o[r] = (_Float16)(s[r] * (float)sc0[idx][r] * inv);
                if (epi == kEpiResidual)
                    o = o + res[idx];  // fp16 add of the rounded product, like the separate kernel
                store_out(o, (size_t)m * N + n);
            }
        }
    }
    if constexpr (CHAIN)
        eet::chain_signal(link);
#if defined(EET_TIMELINE)
    EET_TL_STAMP(3);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    EET_TL_STAMP(4);
    tl_flush();
#endif
#endif
}

struct SmallMConfig {
    int nt, waves, u;
    int ksplit = 1;   // 2: the pair split (nt is 2 then)
};

template <int NT, int RG, int WAVES, int U, bool RMS>
int launch_small_m(const GemmArgs &a)
{
    const int ntiles = a.N / 16;
    dim3 grid((ntiles + NT - 1) / NT), block(WAVES * 64);
    [[maybe_unused]] const int grid_of_launch = (int)grid.x;
    hipLaunchKernelGGL((w8a16_small_m_kernel<NT, RG, WAVES, U, RMS, kPlain>), grid, block, 0, a.st, a.A, a.Wp, a.M, a.N,
                       a.K, a.epi, a.residual, a.rms_gamma, a.scale, a.C, a.rms_eps, eet::ChainLink{}, PairArgs{} EET_TL_ARG);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

// Workspace of a k-split launch: the arrival counters, one per group and 64 bytes apart, in a region of
// fixed size (so that calls of different shapes on one workspace keep their counters in the same, always
// zero, place), then the exchange slots.
constexpr int kSplitMaxGroups = 512;
constexpr size_t kSplitTicketBytes = (size_t)kSplitMaxGroups * 64;
size_t k_split_workspace(int M, int N, int nt, int ks)
{
    const int groups = (N / 16 + nt - 1) / nt, mt = M <= 16 ? 1 : 2;
    return kSplitTicketBytes + (size_t)groups * ks * nt * mt * 1024;
}

// The k split (kernel comment above): NT n-tiles per group of KS workgroups, each a share of the k range.
template <int NT, int RG, int WAVES, int U, int KS>
int launch_small_m_pair(const GemmArgs &a)
{
    const int groups = (a.N / 16 + NT - 1) / NT;
    EET_REQUIRE(groups <= kSplitMaxGroups, EET_ERR_UNSUPPORTED_SHAPE, "eet_gemm_w8a16: the k split takes at most %d groups",
                kSplitMaxGroups);
    EET_REQUIRE(a.ws != nullptr && reinterpret_cast<uintptr_t>(a.ws) % 16 == 0 &&
                    a.ws_bytes >= k_split_workspace(a.M, a.N, NT, KS),
                EET_ERR_WORKSPACE, "eet_gemm_w8a16: the k split needs a 16-byte aligned workspace of %zu bytes, %zu given",
                k_split_workspace(a.M, a.N, NT, KS), a.ws_bytes);
    PairArgs pa;
    pa.tickets = static_cast<unsigned *>(a.ws);
    pa.sums = reinterpret_cast<floatx4 *>(static_cast<char *>(a.ws) + kSplitTicketBytes);
    [[maybe_unused]] const int grid_of_launch = groups * KS;
    hipLaunchKernelGGL((w8a16_small_m_kernel<NT, RG, WAVES, U, false, KS>), dim3(groups, KS), dim3(WAVES * 64), 0, a.st,
                       a.A, a.Wp, a.M, a.N, a.K, a.epi, a.residual, a.rms_gamma, a.scale, a.C, a.rms_eps,
                       eet::ChainLink{}, pa EET_TL_ARG);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

// The chained form: the first launch of a chain is an ordinary launch that signals; a later
// one is issued without the queue barrier and waits in the kernel for its predecessor.
template <int NT, int RG, int WAVES, int U, bool RMS>
int launch_small_m_chained(const GemmArgs &a)
{
    const int ntiles = a.N / 16;
    dim3 grid((ntiles + NT - 1) / NT), block(WAVES * 64);
    eet::ChainLink link;
    bool any_order = false;
    if (int rc = eet::chain_link("eet_gemm_w8a16_chained", a.chain, grid.x, a.st, &link, &any_order))
        return rc;
    auto kern = w8a16_small_m_kernel<NT, RG, WAVES, U, RMS, kChained>;
    if (any_order)
        hipExtLaunchKernelGGL(kern, grid, block, 0, a.st, nullptr, nullptr, hipExtAnyOrderLaunch, a.A, a.Wp, a.M, a.N,
                              a.K, a.epi, a.residual, a.rms_gamma, a.scale, a.C, a.rms_eps, link, PairArgs{} EET_TL_NONE);
    else
        hipLaunchKernelGGL(kern, grid, block, 0, a.st, a.A, a.Wp, a.M, a.N, a.K, a.epi, a.residual, a.rms_gamma,
                           a.scale, a.C, a.rms_eps, link, PairArgs{} EET_TL_NONE);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

// LDS and register budget of an instantiation: the slabs within 64 KiB, the
// reduction buffer (which takes over the slabs' memory when both together pass
// 64 KiB) within 144 of the CU's 160 KiB, and the two register batches small
// enough not to spill.
constexpr bool small_m_fits(int nt, int rg, int waves, int u)
{
    const int mt = (rg + 1) / 2;
    const int stage = waves * u * rg * 1024, red = waves * nt * mt * 1024;
    const int batch_vgprs = 2 * u * (nt + rg) * 4 + nt * mt * 4;
    return stage <= 65536 && red <= 147456 && batch_vgprs <= (waves == 16 ? 96 : 200);
}

// Internal status of dispatch_small_m: no instantiation for this (nt, waves, u) at this row
// count / prologue.  Never crosses the C ABI.
constexpr int kNoVariant = 1;

// Runs the instantiation named by cfg, or with dry = true only tells whether it exists
// (EET_OK / kNoVariant) without launching anything.
template <int RG>
int dispatch_small_m(SmallMConfig cfg, const GemmArgs &a, bool dry)
{
#define EET_CASE(NT_, W_, U_)                                                         \
    if (cfg.nt == NT_ && cfg.waves == W_ && cfg.u == U_) {                            \
        if constexpr (small_m_fits(NT_, RG, W_, U_))                                  \
            return dry ? EET_OK : launch_small_m<NT_, RG, W_, U_, false>(a);          \
    }
#define EET_CASE_RMS(NT_, W_, U_)                                                     \
    if (cfg.nt == NT_ && cfg.waves == W_ && cfg.u == U_) {                            \
        if constexpr (small_m_fits(NT_, RG, W_, U_))                                  \
            return dry ? EET_OK : launch_small_m<NT_, RG, W_, U_, true>(a);           \
    }
    if (cfg.ksplit > 1) {
        // the k split: no RMSnorm prologue, no SwiGLU epilogue, not chained
        if (a.rms_gamma != nullptr || a.epi == kEpiSwiglu || a.chain != eet::kChainOff)
            return kNoVariant;
#define EET_CASE_SPLIT(NT_, W_, U_, KS_)                                                     \
    if (cfg.nt == NT_ && cfg.waves == W_ && cfg.u == U_ && cfg.ksplit == KS_) {              \
        if constexpr (small_m_fits(NT_, RG, W_, U_) && NT_ * ((RG + 1) / 2) <= kPairTiles)   \
            return dry ? EET_OK : launch_small_m_pair<NT_, RG, W_, U_, KS_>(a);              \
    }
        EET_CASE_SPLIT(2, 8, 1, 2) EET_CASE_SPLIT(2, 8, 2, 2) EET_CASE_SPLIT(2, 4, 2, 2)
        EET_CASE_SPLIT(4, 8, 1, 4) EET_CASE_SPLIT(4, 4, 2, 4) EET_CASE_SPLIT(4, 4, 1, 4) EET_CASE_SPLIT(4, 8, 1, 2)
        EET_CASE_SPLIT(5, 8, 1, 4) EET_CASE_SPLIT(5, 4, 2, 4) EET_CASE_SPLIT(5, 4, 1, 4)
        EET_CASE_SPLIT(3, 8, 1, 2) EET_CASE_SPLIT(3, 8, 1, 4) EET_CASE_SPLIT(6, 8, 1, 2)
#undef EET_CASE_SPLIT
        return kNoVariant;
    }
    if (a.chain != eet::kChainOff) {
        // chained kernels exist for the launch shapes pick_small_m can return
#define EET_CASE_CHAIN(NT_, W_, U_)                                                              \
    if (cfg.nt == NT_ && cfg.waves == W_ && cfg.u == U_) {                                        \
        if constexpr (small_m_fits(NT_, RG, W_, U_))                                              \
            return dry ? EET_OK                                                                   \
                       : (a.rms_gamma ? launch_small_m_chained<NT_, RG, W_, U_, true>(a)          \
                                      : launch_small_m_chained<NT_, RG, W_, U_, false>(a));       \
    }
        EET_CASE_CHAIN(1, 8, 2) EET_CASE_CHAIN(1, 16, 2) EET_CASE_CHAIN(1, 16, 1)
        EET_CASE_CHAIN(2, 8, 2) EET_CASE_CHAIN(2, 8, 1) EET_CASE_CHAIN(3, 8, 1)
        EET_CASE_CHAIN(4, 8, 1) EET_CASE_CHAIN(6, 8, 1) EET_CASE_CHAIN(8, 8, 1) EET_CASE_CHAIN(2, 4, 2)
#undef EET_CASE_CHAIN
        return kNoVariant;
    }
    if (a.rms_gamma != nullptr) {
        // the launch shapes pick_small_m can return
        EET_CASE_RMS(1, 8, 2) EET_CASE_RMS(1, 16, 2) EET_CASE_RMS(1, 16, 1)
        EET_CASE_RMS(2, 8, 2) EET_CASE_RMS(2, 8, 1) EET_CASE_RMS(3, 8, 1)
        EET_CASE_RMS(4, 8, 1) EET_CASE_RMS(6, 8, 1) EET_CASE_RMS(8, 8, 1)
        return kNoVariant;
    }
    EET_CASE(1, 4, 4) EET_CASE(1, 8, 4) EET_CASE(1, 16, 4) EET_CASE(1, 8, 2) EET_CASE(1, 16, 2) EET_CASE(1, 16, 1)
    EET_CASE(2, 4, 2) EET_CASE(2, 8, 2) EET_CASE(2, 16, 2) EET_CASE(2, 8, 4) EET_CASE(2, 16, 1) EET_CASE(2, 8, 1)
    EET_CASE(3, 8, 2) EET_CASE(3, 16, 2) EET_CASE(3, 16, 1) EET_CASE(3, 8, 1)
    EET_CASE(4, 4, 2) EET_CASE(4, 8, 2) EET_CASE(4, 8, 1) EET_CASE(4, 16, 1)
    EET_CASE(6, 8, 1) EET_CASE(8, 8, 1)
#undef EET_CASE_RMS
#undef EET_CASE
    return kNoVariant;
}

// Shape -> launch shape: the number of n-tiles per workgroup (NT) that minimises
//   load * (1 + 0.37 * M / (8 * NT)) * (1 + 0.1 / min(4, workgroups / 256))
// where load = ceil(workgroups / 256) * NT is the number of n-tiles the busiest CU
// streams (the kernel is HBM-bound and a CU streams at a fixed rate, so a launch
// of 320 workgroups costs as much as one of 512), the second factor the
// activation traffic (every workgroup reads all M x K activations; they come
// from L2 at about 0.37 of the cost of an HBM byte, 1 KiB per 8 rows and k-tile
// against NT KiB of weights), the third a mild preference for several
// workgroups per CU.  Fitted to sweeps over NT = 1..4, 6, 8 on MI355X at M = 8, 16, 32
// on the LLaMA-7B shapes (N/16 = 768, 256, 1376, 256 n-tiles) and the Baichuan-13B
// shapes (960, 320, 1712, 320), whose order it reproduces: e.g. 1376 n-tiles are 5.4
// per CU, which both NT = 2 (688 workgroups, three rounds) and NT = 6 (230 workgroups,
// one round) turn into a load of 6, the latter with a third of the activation reads
// (M = 32: 20.1 against 28.1 us).  The SwiGLU epilogue needs an even NT (gate / up
// pairs).  One n-tile per workgroup runs with 16 wavefronts when there are few
// workgroups (more loads in flight per CU).
// The k split for the launches without a prologue (O and down projections), where N leaves about one
// n-tile per CU and NT cannot grow without idling CUs.  Measured on MI355X against the table's choice
// (us; residual epilogue; 24 matrices in rotation):
//   N = 4096 (256 n-tiles)            K = 4096: M=16 6.83 -> 6.35 (NT 2, 2 shares)   M=32 8.38 -> 7.38 (NT 2, 2 shares)
//                                     K = 11008: M=16 11.93 -> 10.91 (NT 4, 4 shares) M=32 17.03 -> 13.01 (NT 4, 4 shares)
//                                     M <= 8: no split (5.85 / 9.87 against 6.22 / 10.29)
//   N = 5120 (320 n-tiles, 1.25 per CU: NT 5 with 4 shares makes 256 equal workgroups)
//                                     K = 5120: M=8 7.83 -> 7.67, M=16 9.18 -> 7.94, M=32 11.75 -> 12.29 (not taken)
//                                     K = 13696: M=8 16.43 -> 14.34, M=16 19.53 -> 14.41, M=32 25.27 -> 19.74
// Other channel counts keep the table's choice.
bool pick_k_split(int M, int ntiles, int K, SmallMConfig *out)
{
    if (ntiles == 256 && M > 8) {
        if (K <= 8192)
            *out = M <= 16 ? SmallMConfig{2, 4, 2, 2} : SmallMConfig{2, 8, 1, 2};
        else
            *out = M <= 16 ? SmallMConfig{4, 4, 1, 4} : SmallMConfig{4, 8, 1, 4};
        return true;
    }
    if (ntiles == 320 && !(M > 16 && K <= 8192)) {
        *out = SmallMConfig{5, 8, 1, 4};
        return true;
    }
    return false;
}

// Launch shapes that measured faster than both the formula's choice and the k split on the shapes of the two
// decoders (us per launch, fused prologue / epilogue, 24 or 12 matrices in rotation, formula or split -> this):
//   RMSnorm + QKV, 768 n-tiles (4096 -> 12288): M <= 2  11.33 -> 9.87 with NT 3, i.e. exactly one workgroup per CU
//                                               (the formula takes NT 3 from M = 4 on)
//   RMSnorm + QKV, 960 n-tiles (5120 -> 15360): M = 1 / 2 / 4  16.31 / 14.52 / 14.53 -> 14.75 / 13.76 / 13.89 with NT 2
//                                               and two k-tiles per batch
//   RMSnorm + gate|up, 1712 n-tiles (5120 -> 27392): M <= 2  24.7 -> 23.6 with NT 4; M = 16  26.1 -> 25.4 with NT 8
//   O, 256 n-tiles, K = 4096: M = 1 / 8 / 16  4.94 / 5.21 / 6.03 -> 4.51 / 4.98 / 5.80 with 8 wavefronts and two
//                                               k-tiles per batch instead of 16 wavefronts (M = 16: instead of the split)
//   down, 256 n-tiles, K = 11008: M <= 4  8.81 -> 8.52 with one k-tile per batch
//   O, 320 n-tiles, K = 5120: M = 1 / 4 / 8  7.67 / 7.64 / 7.54 -> 6.34 / 6.72 / 7.31 with NT 2 (160 workgroups of 8
//                                               wavefronts, two k-tiles per batch) instead of the split; M = 32
//                                               11.30 -> 10.95 with 4 wavefronts
bool pick_measured(int M, int ntiles, int K, int epi, bool rms, SmallMConfig *out)
{
    if (rms && epi != kEpiSwiglu) {
        if (ntiles == 768 && M <= 2)
            return *out = SmallMConfig{3, 8, 1}, true;
        if (ntiles == 960 && M <= 4)
            return *out = SmallMConfig{2, 8, 2}, true;
    }
    if (rms && epi == kEpiSwiglu && ntiles == 1712 && M <= 2)
        return *out = SmallMConfig{4, 8, 1}, true;
    if (rms && epi == kEpiSwiglu && ntiles == 1712 && M > 8 && M <= 16)
        return *out = SmallMConfig{8, 8, 1}, true;
    if (!rms && epi != kEpiSwiglu) {
        if (ntiles == 256 && K <= 8192 && M <= 16)
            return *out = SmallMConfig{1, 8, 2}, true;
        if (ntiles == 256 && K > 8192 && M <= 4)
            return *out = SmallMConfig{1, 16, 1}, true;
        if (ntiles == 320 && K <= 8192 && M <= 8)
            return *out = SmallMConfig{2, 8, 2}, true;
        if (ntiles == 320 && K <= 8192 && M > 16)
            return *out = SmallMConfig{2, 4, 2}, true;
    }
    return false;
}

SmallMConfig pick_small_m(int M, int N, int K, int epi, bool rms, bool may_split)
{
    const int ntiles = N / 16;
    if (SmallMConfig measured; pick_measured(M, ntiles, K, epi, rms, &measured))
        return measured;
    if (SmallMConfig split; may_split && !rms && epi != kEpiSwiglu && pick_k_split(M, ntiles, K, &split))
        return split;
    int best_nt = 0;
    double best = 0.0;
    for (int nt : {1, 2, 3, 4, 6, 8}) {
        if (epi == kEpiSwiglu && nt % 2 != 0)
            continue;
        const int wgs = (ntiles + nt - 1) / nt;
        const double load = (double)((wgs + 255) / 256) * nt;
        const double per_cu = wgs / 256.0 < 4.0 ? wgs / 256.0 : 4.0;
        // NT = 6 and 8 leave one workgroup per CU: taken only where they win by more than 3 %
        const double cost = load * (1.0 + 0.37 * M / (8.0 * nt)) * (1.0 + 0.1 / per_cu) * (nt > 4 ? 1.03 : 1.0);
        if (best_nt == 0 || cost < best) {
            best = cost;
            best_nt = nt;
        }
    }
    if (best_nt == 1) {
        const int waves = ntiles >= 512 ? 8 : 16;
        return SmallMConfig{1, waves, M > 16 ? 1 : 2};
    }
    // Two k-tiles per batch only pay where registers allow two resident workgroups:
    // not with the RMSnorm prologue (146 registers with NT = 2: 20.4 us against 17.9 us).
    if (best_nt == 2 && M <= 16 && !rms)
        return SmallMConfig{2, 8, 2};
    return SmallMConfig{best_nt, 8, 1};
}

int dispatch_by_rows(SmallMConfig cfg, const GemmArgs &a, bool dry)
{
    if (a.M <= 8)
        return dispatch_small_m<1>(cfg, a, dry);
    if (a.M <= 16)
        return dispatch_small_m<2>(cfg, a, dry);
    return dispatch_small_m<4>(cfg, a, dry);
}

// The launch shape a call runs with: the tuning override when an instantiation of that shape
// exists for this call (decided without launching), otherwise the table's choice.
SmallMConfig resolve_small_m(const GemmArgs &a)
{
    const eet::Tuning &tune = eet::tuning();
    if (tune.has_small_m && (a.epi != kEpiSwiglu || tune.small_m_nt % 2 == 0)) {
        const SmallMConfig forced{tune.small_m_nt, tune.small_m_waves, tune.small_m_u, tune.small_m_ksplit};
        if (dispatch_by_rows(forced, a, true) == EET_OK)
            return forced;
    }
    // the k split runs out of the caller's workspace: without a sufficient one the table's choice stands
    SmallMConfig cfg = pick_small_m(a.M, a.N, a.K, a.epi, a.rms_gamma != nullptr, a.chain == eet::kChainOff);
    if (cfg.ksplit > 1 && (a.ws == nullptr || reinterpret_cast<uintptr_t>(a.ws) % 16 != 0 ||
                           a.ws_bytes < k_split_workspace(a.M, a.N, cfg.nt, cfg.ksplit)))
        cfg = pick_small_m(a.M, a.N, a.K, a.epi, a.rms_gamma != nullptr, false);
    return cfg;
}

int run_small_m(const GemmArgs &a)
{
    // the kernel addresses the packed weights through one buffer resource with 32-bit offsets
    if ((size_t)a.K * a.N >= (1ull << 31))
        return eet::fail(EET_ERR_UNSUPPORTED_SHAPE, "eet_gemm_w8a16: K x N = %d x %d exceeds the 2 GiB weight limit",
                         a.K, a.N);
    const SmallMConfig cfg = resolve_small_m(a);
    const int rc = dispatch_by_rows(cfg, a, false);   // a launch failure is returned as it is
    if (rc == kNoVariant)
        return eet::fail(EET_ERR_INVALID_ARGUMENT,
                         "eet_gemm_w8a16: no small-M kernel for nt=%d waves=%d u=%d ksplit=%d (M=%d%s)", cfg.nt, cfg.waves,
                         cfg.u, cfg.ksplit, a.M, a.rms_gamma ? ", RMSnorm prologue" : "");
    return rc;
}

}  // namespace

// 33 <= M <= 64 with few channels: see run_gemm.
static bool takes_slabs(int M, int N)
{
    const int tile_wgs = ((M + 31) / 32) * ((N + 127) / 128);
    return M <= 64 && tile_wgs < 150;
}

static int run_gemm(const GemmArgs &a)
{
    if (a.M <= 32)
        return run_small_m(a);
    // 33 <= M <= 64 with few channels and no workspace to split the k range with: the 32 x 128
    // MFMA tiles would number under ~150 and each would walk the whole k range alone (19 us at
    // N = 4096, K = 4096 whatever M is), so the small-M kernel runs over 32-row slabs instead
    // (12-15 us; the weights are re-read per slab, from L2 / Infinity Cache).  With the workspace
    // the split MFMA launch is faster still (10-11 us; 16 against 24-34 us at K = 11008).
    const size_t split_bytes = eet::large_m_workspace(a.M, a.N, a.K, a.epi);
    const bool can_split = split_bytes > 0 && a.ws != nullptr && a.ws_bytes >= split_bytes &&
                           reinterpret_cast<uintptr_t>(a.ws) % 16 == 0;
    if (takes_slabs(a.M, a.N) && !can_split && !eet::tuning().has_large_m) {
        const int n_out = (a.epi == kEpiSwiglu) ? a.N / 2 : a.N;
        for (int m0 = 0; m0 < a.M; m0 += 32) {
            GemmArgs s = a;
            s.M = (a.M - m0 < 32) ? a.M - m0 : 32;
            s.A = a.A + (size_t)m0 * a.K;
            s.C = a.C + (size_t)m0 * n_out;
            if (a.residual)
                s.residual = a.residual + (size_t)m0 * a.N;
            if (int rc = run_small_m(s))
                return rc;
        }
        return EET_OK;
    }
    return eet::run_large_m(a);
}

static int check_gemm_args(const char *fn, const void *A, const void *W, const void *scale, const void *C, int M,
                           int N, int K)
{
    EET_REQUIRE(A && W && scale && C, EET_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    EET_REQUIRE(M >= 0 && N > 0 && K > 0, EET_ERR_INVALID_ARGUMENT, "%s: bad sizes M=%d N=%d K=%d", fn, M, N, K);
    EET_REQUIRE(K % 64 == 0 && N % 16 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "%s: need K %% 64 == 0 and N %% 16 == 0, got K=%d N=%d", fn, K, N);
    EET_REQUIRE((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) % 16 == 0 &&
                    (reinterpret_cast<uintptr_t>(scale) | reinterpret_cast<uintptr_t>(C)) % 8 == 0,
                EET_ERR_INVALID_ARGUMENT, "%s: A and W must be 16-byte aligned, scale and C 8-byte", fn);
    return EET_OK;
}

extern "C" int eet_gemm_w8a16(const void *A, const void *Wpacked, const void *scale, void *C, int M, int N, int K,
                              void *workspace, size_t workspace_bytes, void *stream)
{
    if (int rc = check_gemm_args("eet_gemm_w8a16", A, Wpacked, scale, C, M, N, K))
        return rc;
    if (M == 0)
        return EET_OK;
    return run_gemm(GemmArgs{static_cast<const _Float16 *>(A), static_cast<const u32x4 *>(Wpacked),
                             static_cast<const _Float16 *>(scale), static_cast<_Float16 *>(C), M, N, K, nullptr,
                             kEpiNone, nullptr, 0.f, workspace, workspace_bytes, static_cast<hipStream_t>(stream)});
}

extern "C" int eet_gemm_w8a16_small_m_shape(int M, int N, int K, int epilogue, int rms_prologue, int *nt, int *waves,
                                            int *k_tiles_per_batch, int *k_split)
{
    EET_REQUIRE(nt && waves && k_tiles_per_batch && k_split, EET_ERR_INVALID_ARGUMENT,
                "eet_gemm_w8a16_small_m_shape: null pointer");
    EET_REQUIRE(M >= 1 && M <= 32 && N > 0 && K > 0 && K % 64 == 0 && N % 16 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_gemm_w8a16_small_m_shape: not a shape the small-M kernel takes (M=%d N=%d K=%d)", M, N, K);
    GemmArgs a{};
    a.M = M, a.N = N, a.K = K, a.epi = epilogue;
    static const _Float16 kSomeGamma = 0;
    a.rms_gamma = rms_prologue ? &kSomeGamma : nullptr;   // only tested against null
    // as for a call that hands over the workspace eet_gemm_w8a16_workspace asks for (never dereferenced here)
    static const u32x4 kSomeWorkspace = {0, 0, 0, 0};
    a.ws = const_cast<u32x4 *>(&kSomeWorkspace);
    a.ws_bytes = ~size_t(0);
    const SmallMConfig cfg = resolve_small_m(a);
    *nt = cfg.nt, *waves = cfg.waves, *k_tiles_per_batch = cfg.u, *k_split = cfg.ksplit;
    // The library must hold a kernel for what the table answers in every form of the call: with the
    // workspace (above), without it, and chained.  Decided without launching.
    GemmArgs bare = a, chained = a;
    bare.ws = nullptr, bare.ws_bytes = 0;
    chained.ws = nullptr, chained.ws_bytes = 0, chained.chain = eet::kChainNext;
    for (const GemmArgs *form : {&a, &bare, &chained}) {
        const SmallMConfig c = resolve_small_m(*form);
        EET_REQUIRE(dispatch_by_rows(c, *form, true) == EET_OK, EET_ERR_INVALID_ARGUMENT,
                    "eet_gemm_w8a16_small_m_shape: no small-M kernel for nt=%d waves=%d u=%d ksplit=%d (M=%d N=%d K=%d epilogue %d%s%s)",
                    c.nt, c.waves, c.u, c.ksplit, M, N, K, epilogue, rms_prologue ? ", RMSnorm prologue" : "",
                    form == &chained ? ", chained" : form == &bare ? ", no workspace" : "");
    }
    return EET_OK;
}

extern "C" size_t eet_gemm_w8a16_workspace(int M, int N, int K, int epilogue)
{
    if (M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || N % 16 != 0)
        return 0;
    if (M <= 32) {   // the small-M kernel's k split (launches without the RMSnorm prologue)
        const eet::Tuning &tune = eet::tuning();
        SmallMConfig cfg = pick_small_m(M, N, K, epilogue, false, true);
        if (tune.has_small_m && tune.small_m_ksplit > 1)
            cfg = SmallMConfig{tune.small_m_nt, tune.small_m_waves, tune.small_m_u, tune.small_m_ksplit};
        return cfg.ksplit > 1 ? k_split_workspace(M, N, cfg.nt, cfg.ksplit) : 0;
    }
    return eet::large_m_workspace(M, N, K, epilogue);
}

static int gemm_fused(const char *fn, const void *A, const void *Wpacked, const void *scale, void *C, int M, int N,
                      int K, int epilogue, const void *residual, const void *rms_gamma, float rms_eps,
                      void *workspace, size_t workspace_bytes, int chain, void *stream)
{
    if (int rc = check_gemm_args(fn, A, Wpacked, scale, C, M, N, K))
        return rc;
    EET_REQUIRE(epilogue == EET_EPILOGUE_NONE || epilogue == EET_EPILOGUE_RESIDUAL || epilogue == EET_EPILOGUE_SWIGLU,
                EET_ERR_INVALID_ARGUMENT, "%s: unknown epilogue %d", fn, epilogue);
    EET_REQUIRE((epilogue == EET_EPILOGUE_RESIDUAL) == (residual != nullptr), EET_ERR_INVALID_ARGUMENT,
                "%s: residual must be given exactly for EET_EPILOGUE_RESIDUAL", fn);
    EET_REQUIRE(residual == nullptr || reinterpret_cast<uintptr_t>(residual) % 8 == 0, EET_ERR_INVALID_ARGUMENT,
                "%s: residual must be 8-byte aligned", fn);
    EET_REQUIRE(epilogue != EET_EPILOGUE_SWIGLU || N % 32 == 0, EET_ERR_UNSUPPORTED_SHAPE,
                "%s: the SwiGLU epilogue needs N %% 32 == 0 (gate/up tile pairs), got N=%d", fn, N);
    EET_REQUIRE(rms_gamma == nullptr || (M <= 32 && reinterpret_cast<uintptr_t>(rms_gamma) % 16 == 0),
                EET_ERR_UNSUPPORTED_SHAPE,
                "%s: the RMSnorm prologue is available for M <= 32 only (M=%d) and needs a 16-byte aligned gamma", fn,
                M);
    EET_REQUIRE(chain == eet::kChainOff || chain == eet::kChainFirst || chain == eet::kChainNext,
                EET_ERR_INVALID_ARGUMENT, "%s: unknown chain mode %d", fn, chain);
    EET_REQUIRE(chain == eet::kChainOff || (M >= 1 && M <= 32), EET_ERR_UNSUPPORTED_SHAPE,
                "%s: chained launches exist for 1 <= M <= 32 only (M=%d)", fn, M);
    if (M == 0)
        return EET_OK;
    GemmArgs args{static_cast<const _Float16 *>(A), static_cast<const u32x4 *>(Wpacked),
                  static_cast<const _Float16 *>(scale), static_cast<_Float16 *>(C), M, N, K,
                  static_cast<const _Float16 *>(residual), epilogue, static_cast<const _Float16 *>(rms_gamma), rms_eps,
                  workspace, workspace_bytes, static_cast<hipStream_t>(stream)};
    args.chain = chain;
    return run_gemm(args);
}

extern "C" int eet_gemm_w8a16_fused(const void *A, const void *Wpacked, const void *scale, void *C, int M, int N,
                                    int K, int epilogue, const void *residual, const void *rms_gamma, float rms_eps,
                                    void *workspace, size_t workspace_bytes, void *stream)
{
    return gemm_fused("eet_gemm_w8a16_fused", A, Wpacked, scale, C, M, N, K, epilogue, residual, rms_gamma, rms_eps,
                      workspace, workspace_bytes, eet::kChainOff, stream);
}

extern "C" int eet_gemm_w8a16_chained(const void *A, const void *Wpacked, const void *scale, void *C, int M, int N,
                                      int K, int epilogue, const void *residual, const void *rms_gamma, float rms_eps,
                                      int chain, void *stream)
{
    return gemm_fused("eet_gemm_w8a16_chained", A, Wpacked, scale, C, M, N, K, epilogue, residual, rms_gamma, rms_eps,
                      nullptr, 0, chain, stream);
}

#if defined(EET_TIMELINE)
// Bench-only: recording starts with a device buffer for `launches` launches; every small-M launch made through the
// eet_timeline_* entry points from then on fills the next slot.  eet_timeline_read synchronises the device, copies
// slot `launch` ([workgroup][24]: 8 clock readings of the 100 MHz wall clock: entry, first batch multiplied, k loop
// done, stores issued, stores acknowledged) and returns the workgroup count of that launch, or a negative value.
extern "C" int eet_timeline_begin(int launches)
{
    if (g_tl_buf != nullptr && g_tl_cap < launches) {
        (void)hipFree(g_tl_buf);
        g_tl_buf = nullptr;
    }
    if (g_tl_buf == nullptr) {
        EET_HIP_CHECK(hipMalloc(&g_tl_buf, (size_t)launches * kTlMaxWgs * kTlStamps * sizeof(unsigned long long)));
        g_tl_cap = launches;
    }
    EET_HIP_CHECK(hipMemset(g_tl_buf, 0, (size_t)g_tl_cap * kTlMaxWgs * kTlStamps * sizeof(unsigned long long)));
    g_tl_n = 0;
    return EET_OK;
}

extern "C" int eet_timeline_launches(void) { return g_tl_n; }

extern "C" int eet_timeline_read(int launch, unsigned long long *host_dst)
{
    if (launch < 0 || launch >= g_tl_n || host_dst == nullptr)
        return -1;
    if (hipDeviceSynchronize() != hipSuccess)
        return -2;
    const int wgs = g_tl_grid[launch];
    if (hipMemcpy(host_dst, g_tl_buf + (size_t)launch * kTlMaxWgs * kTlStamps, (size_t)wgs * kTlStamps * sizeof(unsigned long long),
                  hipMemcpyDeviceToHost) != hipSuccess)
        return -2;
    return wgs;
}
#endif
