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
#include <type_traits>

#include "common.h"
#include "tuning.h"

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

// Maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 with the lane-swap instructions of gfx950 (two vector
// instructions per step, no trip through the LDS crossbar as a bpermute takes).  v_permlane16_swap exchanges the
// odd 16-lane rows of its first operand with the even rows of its second: on two copies of v it leaves (even rows
// duplicated, odd rows duplicated); v_permlane32_swap does the same with the two 32-lane halves.  Written as
// assembly because the compiler builtin dropped the second result; the s_nop's cover the wait states the
// instruction needs after a vector write of its operands and before a vector read of its results.
__device__ __forceinline__ float max_over_lane_groups(float v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    float x = v, y = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));
    x = y = fmaxf(x, y);
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x), "+v"(y));
    v = fmaxf(x, y);
#endif
    return v;
}

// Which (batch, head) pair and query block a workgroup takes.  Workgroup i runs on XCD i % 8 and the XCDs have an
// L2 each, so the workgroups that are resident on an XCD at one time should be the query blocks of FEW pairs: they
// walk the same K and V rows at about the same time and fetch each of them once between them.  With `group` > 0
// and a pair count divisible by 8, XCD x owns the pairs x, x + 8, ... in groups of `group`; inside a group the
// longest (last) query block of every pair is handed out first, then the one before (the long blocks start first,
// the short ones fill the tail, group after group).  group = 0: all pairs of the last query block first, then
// those of the one before, over the whole launch (every resident workgroup then has a pair of its own, and a
// prompt's K and V cross the fabric once per query block instead of once).
__device__ __forceinline__ void prefill_block_of(int group, int *bh, int *qblock)
{
    const int pairs = gridDim.x, q_blocks = gridDim.y;
    if (group <= 0 || pairs % 8 != 0) {
        *bh = blockIdx.x;
        *qblock = q_blocks - 1 - (int)blockIdx.y;
        return;
    }
    const int lin = blockIdx.y * pairs + blockIdx.x;
    const int xcd = lin % 8, q = lin / 8, per_xcd = pairs / 8;
    const int gs = group * q_blocks, g = q / gs, r = q % gs;
    const int gl = min(group, per_xcd - g * group);       // pairs of this group (the last may be smaller)
    *bh = (g * group + r % gl) * 8 + xcd;
    *qblock = q_blocks - 1 - r / gl;
}

template <int DH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) void prefill_attention_kernel(
    const _Float16 *__restrict__ q, const _Float16 *__restrict__ k_cache, const _Float16 *__restrict__ v_cache,
    _Float16 *__restrict__ ctx, const _Float16 *__restrict__ alibi, const int64_t *__restrict__ pad, int H, int S,
    int T_cap, float scale, int group)
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
    int bh, qblock;
    prefill_block_of(group, &bh, &qblock);
    const int b = bh / H, h = bh % H;
    const int q0 = qblock * kBQ;
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
                for (int r = 0; r < 4; ++r)
                    sacc[qt][kt][r] = sacc[qt][kt][r] * scale2 + (float)bias4[kt][r] * kLog2e;
            // one branch around all sixteen tests (inside the loop above it becomes a branch per score)
            if (need_mask) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = kc0 + 16 * kt + 4 * g + r;
                        sacc[qt][kt][r] = (key > qi || key < padb) ? -INFINITY : sacc[qt][kt][r];
                    }
            }
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    cmax = fmaxf(cmax, sacc[qt][kt][r]);
            cmax = max_over_lane_groups(cmax);
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
            // the accumulator is rescaled only when some query's maximum moved (rare after the first chunks)
            if (__builtin_amdgcn_ballot_w64(corr != 1.0f) != 0) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    oacc[qt][dt] *= corr;
            }
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


// ---------------------------------------------------------------------------
// Head size 128 (LLaMA-7B, Baichuan-13B): the same transposed formulation with
// the K and V chunks brought into LDS by the memory pipeline itself.
//
// A workgroup of 8 wavefronts takes 256 queries of one (b, h); wavefront w owns
// the 16-query tiles w and w + 8 of the block (one early, one late, so that the
// causal triangle is split evenly) and skips a tile once the chunks have passed
// its diagonal.  K and V rows stay row-major in LDS, 256 B per row, copied
// global -> LDS with buffer_load_dwordx4 ... lds (no staging registers, no
// ds_write) into a ring of four 64-key stages, one pair of chunks ahead of the
// pair being multiplied; one s_barrier per pair.  Piece p (16 B) of row r sits at
// position p ^ swz(r), with one swizzle for K and another for V, so that the K
// operand reads (lane = row) and the V reads hit distinct banks.  V^T operands come out of the row-major rows through
// ds_read_b64_tr_b16, which hands lane i column i of a 4 x 16 block of halves.
// ---------------------------------------------------------------------------
constexpr int kD = 128;

constexpr int kKAhead = 6, kVAhead = 4;    // K operand reads / V operands (two reads each) in flight ahead of their MFMAs
constexpr int kStageVec = 2 * 1024 + 16;   // u32x4 per stage: K rows, V rows, bias row (+ padding)

// Measured on MI355X with 8 wavefronts reading back to back: a 16-byte operand read (lane = row) runs at
// full rate when the piece index is XORed with the row number itself, and at half rate with the V
// swizzle or with rows padded to 272 B; the transposing 8-byte reads of V run at full rate with the
// swizzle below (4 consecutive rows must land on 4 different pairs of positions) and not with padding.
__device__ __forceinline__ int k_swz(int r) { return r & 15; }
__device__ __forceinline__ int row_swz(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }

typedef short short4v __attribute__((ext_vector_type(4)));

// NQT 16-query tiles per wavefront, WAVES wavefronts, STAGES chunk buffers: 16 NQT WAVES queries per workgroup.
// <2, 8, 4>: two wavefronts per SIMD with 256 registers each, every K and V operand read feeds two tiles;
// <1, 8, 2>: half the queries and half the ring, so that two workgroups fit a CU, four wavefronts per SIMD, twice
// the operand reads per query (the LDS has the room).  launch_dh128 says which runs when.
template <bool ALIBI, int NQT, int WAVES, int STAGES>
__global__ __launch_bounds__(64 * WAVES)
    __attribute__((amdgpu_waves_per_eu(STAGES == 2 ? 2 * WAVES / 4 : WAVES / 4, STAGES == 2 ? 2 * WAVES / 4 : WAVES / 4))) void prefill_attention_dh128_kernel(
    const _Float16 *__restrict__ q, const _Float16 *__restrict__ k_cache, const _Float16 *__restrict__ v_cache,
    _Float16 *__restrict__ ctx, const _Float16 *__restrict__ alibi, const int64_t *__restrict__ pad, int H, int S,
    int T_cap, float scale, int group)
{
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    constexpr int DC = kD / 32, DT = kD / 16;
    constexpr int kBQ2 = 16 * NQT * WAVES;   // queries per workgroup
    constexpr int kGroup = STAGES / 2;       // chunks per barrier
    __shared__ u32x4 lds[STAGES * kStageVec];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, j = lane & 15;
    // Workgroups take (pair, query block) in the order of prefill_block_of: long blocks before short ones (with the
    // block index running fastest the last CU to finish held up to a fifth of the launch), few pairs per XCD at a time.
    int bh, qblock;
    prefill_block_of(group, &bh, &qblock);
    const int b = bh / H, h = bh % H;
    const int q0 = qblock * kBQ2;
    const int padb = pad ? (int)min((int64_t)S, max((int64_t)0, pad[b])) : 0;

    const _Float16 *kbase = k_cache + (size_t)bh * T_cap * kD;
    const _Float16 *vbase = v_cache + (size_t)bh * T_cap * kD;
    const _Float16 *qbase = q + (size_t)bh * S * kD;
    // rows >= S are out of range: they read as zeros (and are masked: such a key follows every query)
    const __amdgpu_buffer_rsrc_t krs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(kbase), 0, (unsigned)S * (kD * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(vbase), 0, (unsigned)S * (kD * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(ALIBI ? alibi + (size_t)h * S : q), 0, ALIBI ? (unsigned)S * 2u : 0u, 0x00020000);

    static_assert((NQT == 1 || NQT == 2) && 16 % WAVES == 0 && (STAGES == 2 || STAGES == 4), "launch shape");
    constexpr int KI = 16 / WAVES;   // DMA instructions per wavefront for the K rows of a chunk (and for the V rows)
    // the query tiles of this wavefront: one early, one late (the causal triangle is split evenly)
    int tq0[NQT];
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt)
        tq0[qt] = q0 + 16 * (wave + qt * WAVES);
    half8 qop[NQT][DC];
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        const int qi = min(tq0[qt] + j, S - 1);
#pragma unroll
        for (int c = 0; c < DC; ++c)
            qop[qt][c] = *reinterpret_cast<const half8 *>(qbase + (size_t)qi * kD + 32 * c + 8 * g);
    }
    floatx4 oacc[NQT][DT];
    // The softmax denominators ride along as one more accumulator tile per query tile: P^T times a V^T operand of
    // ones leaves, in every row, the sum over the keys of the weights as the matrix cores see them (rounded to
    // fp16, like the numerator) -- two matrix instructions per chunk and tile instead of sixteen vector adds per
    // lane, and no cross-lane sum at the end.
    floatx4 lacc[NQT];
    float m_run[NQT];
    const half8 ones8 = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f,
                         (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        m_run[qt] = -INFINITY;
        lacc[qt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            oacc[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    // DMA: instruction t of a chunk fills rows 4t .. 4t+3 (1 KiB); lane l carries position l % 16 of row
    // 4t + l / 16, i.e. piece (l % 16) ^ swz(row).  Wavefront w issues instructions KI w .. KI w + KI - 1 of K and of V.
    int dma_off_k[KI], dma_off_v[KI];   // byte offset of this lane's piece within a chunk, per instruction
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int row = 4 * (KI * wave + i) + (lane >> 4);
        dma_off_k[i] = row * (kD * 2) + (((lane & 15) ^ k_swz(row)) << 4);
        dma_off_v[i] = row * (kD * 2) + (((lane & 15) ^ row_swz(row)) << 4);
    }
    auto dma_chunk = [&](int stage, int kc0) {
        u32x4 *st = lds + stage * kStageVec;
        const int base = kc0 * (kD * 2);   // in the lane offset: the range check of a buffer load covers it
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(krs, st + (KI * wave + i) * 64, 16, base + dma_off_k[i], 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(vrs, st + 1024 + (KI * wave + i) * 64, 16, base + dma_off_v[i], 0, 0, 0);
        }
        if (ALIBI)   // the chunk's 64 bias terms (128 B): every wavefront writes the same bytes
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ars, st + 2048, 4, kc0 * 2 + (lane & 31) * 4, 0, 0, 0);
    };

    constexpr float kLog2e = 1.4426950408889634f;
    constexpr float kLazy = 8.0f;   // in powers of two
    const float scale2 = scale * kLog2e;
    const int k_begin = (padb / kBK) * kBK;
    const int k_end = min(S, q0 + kBQ2);
    const int nchunks = (k_end - k_begin + kBK - 1) / kBK;

    // the work on one chunk for the query tiles named in MASK (bit qt)
    auto compute = [&](auto mask_c, const u32x4 *st, int kc0) {
        constexpr int MASK = decltype(mask_c)::value;
        const u32x4 *kst = st;
        const unsigned char *vst = reinterpret_cast<const unsigned char *>(st + 1024);
        floatx4 sacc[NQT][4];
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt)
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                sacc[qt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            const int row = 16 * kt + j;
#pragma unroll
            for (int c = 0; c < DC; ++c) {
                const half8 kop = __builtin_bit_cast(half8, kst[row * 16 + ((4 * c + g) ^ k_swz(row))]);
#pragma unroll
                for (int qt = 0; qt < NQT; ++qt)
                    if (MASK & (1 << qt))
                        sacc[qt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop, qop[qt][c], sacc[qt][kt], 0, 0, 0);
            }
        }
        // operand reads kKAhead ahead of the matrix instructions that use them (six against three: +5 % on a
        // 2048-token prompt, two: -8 %)
        {
            constexpr int kPer = (MASK == 3) ? 2 : 1;   // query tiles taking part
            __builtin_amdgcn_sched_group_barrier(0x100, kKAhead, 0);
#pragma unroll
            for (int n = 0; n < 16 - kKAhead; ++n) {
                __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, kKAhead * kPer, 0);
        }
        half4 bias4[4];
        if (ALIBI) {
            const _Float16 *bst = reinterpret_cast<const _Float16 *>(st + 2048);
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
                bias4[kt] = *reinterpret_cast<const half4 *>(bst + 16 * kt + 4 * g);
        }
        half8 pop[NQT][2];
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
            if (!(MASK & (1 << qt)))
                continue;
            const int qi = tq0[qt] + j;
            float cmax = -INFINITY;
            const bool need_mask = (kc0 + kBK - 1 > tq0[qt]) || (kc0 < padb);
            // Without a bias the scale is applied inside the exponent's argument (one fused multiply-add per
            // element instead of a multiply and a subtract): the maximum is taken over the raw products and
            // scaled once (the scale is positive).
            if (ALIBI) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        sacc[qt][kt][r] = sacc[qt][kt][r] * scale2 + (float)bias4[kt][r] * kLog2e;
            }
            // one branch around all sixteen tests (inside the loop below it became a branch per score)
            if (need_mask) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = kc0 + 16 * kt + 4 * g + r;
                        sacc[qt][kt][r] = (key > qi || key < padb) ? -INFINITY : sacc[qt][kt][r];
                    }
            }
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    cmax = fmaxf(cmax, sacc[qt][kt][r]);
            cmax = max_over_lane_groups(cmax);
            if (!ALIBI)
                cmax *= scale2;
            // m_run is the reference exponent of the query: it follows the maximum lazily, only when a chunk's
            // maximum passes it by more than kLazy (then the accumulators are rescaled; rare after a query's first
            // chunk, where following every new maximum rescaled in most chunks of a short prompt).  Weights reach
            // 2^kLazy at most, well inside fp16, and numerator and denominator share the reference.
            const float m_ref = m_run[qt];
            const bool raise = cmax > m_ref + kLazy;   // also the first keys of the query: m_ref is -inf
            if (__builtin_amdgcn_ballot_w64(raise) != 0) {
                const float corr = raise ? __builtin_amdgcn_exp2f(m_ref - cmax) : 1.0f;   // 0 for the first keys
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    oacc[qt][dt] *= corr;
                lacc[qt] *= corr;
                m_run[qt] = raise ? cmax : m_ref;
            }
            const float m_safe = (m_run[qt] == -INFINITY) ? 0.f : m_run[qt];
            float p[4][4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    p[kt][r] = ALIBI ? __builtin_amdgcn_exp2f(sacc[qt][kt][r] - m_safe)
                                     : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[qt][kt][r], scale2, -m_safe));
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
        // O^T += V^T . P^T.  Lane (g, j) needs d = 16*dt + j and keys 4g .. 4g+3 of tiles 2*hf and 2*hf + 1.
        // One transposing read covers the 4 keys of one tile: lane j of a 16-lane group supplies 8 bytes
        // (d = 16*dt + 4*(j%4) .. +3) of key row 4g + j/4 and receives the column d = 16*dt + j.
        const int vr = j >> 2, vc4 = j & 3;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                short4v part[2];
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const int key = 32 * hf + 16 * a + 4 * g + vr;
                    const int pos = (2 * dt + (vc4 >> 1)) ^ row_swz(key);
                    const unsigned char *addr = vst + key * (kD * 2) + pos * 16 + (vc4 & 1) * 8;
                    part[a] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (short4v __attribute__((address_space(3))) *)(addr));
                }
                const half4 lo = __builtin_bit_cast(half4, part[0]), hi = __builtin_bit_cast(half4, part[1]);
                const half8 vop = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int qt = 0; qt < NQT; ++qt)
                    if (MASK & (1 << qt))
                        oacc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vop, pop[qt][hf], oacc[qt][dt], 0, 0, 0);
            }
        }
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int qt = 0; qt < NQT; ++qt)
                if (MASK & (1 << qt))
                    lacc[qt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones8, pop[qt][hf], lacc[qt], 0, 0, 0);
        // the transposing reads (two per operand) kVAhead operands ahead of the matrix instructions
        {
            constexpr int kPer = (MASK == 3) ? 2 : 1;   // query tiles taking part
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * kVAhead, 0);
#pragma unroll
            for (int n = 0; n < 2 * DT - kVAhead; ++n) {
                __builtin_amdgcn_sched_group_barrier(0x008, kPer, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, (kVAhead + 2) * kPer, 0);   // + the two of the denominators
        }
    };

    auto chunk = [&](int c) {
        const int kc0 = k_begin + c * kBK;
        const u32x4 *st = lds + (c % STAGES) * kStageVec;
        const bool t0 = kc0 <= tq0[0] + 15 && tq0[0] < S;
        const bool t1 = NQT == 2 && kc0 <= tq0[NQT - 1] + 15 && tq0[NQT - 1] < S;
        if (t0 && t1)
            compute(std::integral_constant<int, NQT == 2 ? 3 : 1>{}, st, kc0);
        else if (t1)
            compute(std::integral_constant<int, NQT == 2 ? 2 : 1>{}, st, kc0);
        else if (t0)
            compute(std::integral_constant<int, 1>{}, st, kc0);
    };
    // kGroup chunks per barrier (two with four stages, one with two): while one group is multiplied the next is on
    // its way into the other half of the ring.  (A chunk past the end reads rows >= S: zeros, no memory touched
    // beyond the range; past k_end but below S it is a wasted copy.)
#pragma unroll
    for (int gi = 0; gi < kGroup; ++gi)
        dma_chunk(gi, k_begin + gi * kBK);
    for (int c0 = 0; c0 < nchunks; c0 += kGroup) {
        // everything requested so far is this iteration's group of chunks
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int gi = 0; gi < kGroup; ++gi)   // these stages were read in the iteration before
            dma_chunk((c0 + kGroup + gi) % STAGES, k_begin + (c0 + kGroup + gi) * kBK);
#pragma unroll
        for (int gi = 0; gi < kGroup; ++gi)
            if (c0 + gi < nchunks)
                chunk(c0 + gi);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no copy may land in LDS after the workgroup has gone

#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        const float l = lacc[qt][0];   // every row of the tile holds the sum for query j
        const int qi = tq0[qt] + j;
        if (qi >= S)
            continue;
        const float inv = (qi < padb) ? 0.f : 1.0f / (l + 1e-6f);
        _Float16 *dst = ctx + ((size_t)(b * S + qi) * H + h) * kD;
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

// Pairs per XCD group (prefill_block_of): as many as fill the workgroup slots of an XCD with all their query
// blocks, at least four (measured at B*H = 256 .. 1280, 512 .. 8192 tokens: 4 .. 16 pairs are within noise of one
// another and 5-12 % ahead of the ungrouped order; one or two pairs lose to it, their long blocks idle too many CUs
// while they finish).  A launch that fits the slots in one round keeps the ungrouped order: there the dispatcher
// pairs workgroup i with workgroup i + 32 on a CU, and only that order makes it a long block with a short one.
// The tuning key EET_PREFILL_GROUP forces a count, -1 the ungrouped order.
int pairs_per_group(int slots_per_xcd, int q_blocks, int pairs)
{
    const int forced = eet::tuning().prefill_group;
    if (forced != 0)
        return forced < 0 ? 0 : forced;
    if (q_blocks < 1 || pairs % 8 != 0 || (pairs / 8) * q_blocks <= slots_per_xcd)
        return 0;
    const int g = slots_per_xcd / q_blocks;
    return g < 4 ? 4 : g;
}

int launch_dh128(const void *q, const void *kc, const void *vc, void *ctx, const void *alibi, const int64_t *pad, int B,
                 int H, int S, int T_cap, hipStream_t st)
{
    const float scale = (float)(_Float16)(1.0f / sqrtf(128.0f));
    // Launch shape by prompt length (measured at B*H = 256 .. 320):
    //   1  128 queries per workgroup, eight one-tile wavefronts, two stages: two workgroups share a CU, so the
    //      start-up, the diagonal chunks and the drain of one overlap the other's work -- up to 1536 tokens
    //      (+13 % at 256, +20 % at 512, +6-9 % at 1024, +2-3 % at 1536; 3-6 % behind from 2048 on);
    //   2  256 queries, eight two-tile wavefronts, four stages (every operand read feeds two tiles) -- beyond.
    // (256 queries as sixteen one-tile wavefronts was within 2 % of shape 2 everywhere and is not kept.)
    // A tuning override picks either.
    int shape = eet::tuning().prefill_shape;
    if (shape < 1 || shape > 2)
        shape = S <= 1536 ? 1 : 2;
#define EET_PF_LAUNCH(A_, N_, W_, S_)                                                                              \
    hipLaunchKernelGGL((prefill_attention_dh128_kernel<A_, N_, W_, S_>),                                          \
                       dim3(B * H, (S + 16 * N_ * W_ - 1) / (16 * N_ * W_)), dim3(64 * W_), 0, st,                \
                       static_cast<const _Float16 *>(q), static_cast<const _Float16 *>(kc),                       \
                       static_cast<const _Float16 *>(vc), static_cast<_Float16 *>(ctx),                           \
                       static_cast<const _Float16 *>(alibi), pad, H, S, T_cap, scale,                             \
                       pairs_per_group(32 * (shape == 1 ? 2 : 1), (S + 16 * N_ * W_ - 1) / (16 * N_ * W_), B * H))
    if (alibi != nullptr) {
        if (shape == 1)
            EET_PF_LAUNCH(true, 1, 8, 2);
        else
            EET_PF_LAUNCH(true, 2, 8, 4);
    } else {
        if (shape == 1)
            EET_PF_LAUNCH(false, 1, 8, 2);
        else
            EET_PF_LAUNCH(false, 2, 8, 4);
    }
#undef EET_PF_LAUNCH
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

template <int DH>
int launch(const void *q, const void *kc, const void *vc, void *ctx, const void *alibi, const int64_t *pad, int B,
           int H, int S, int T_cap, hipStream_t st)
{
    const float scale = (float)(_Float16)(1.0f / sqrtf((float)DH));
    dim3 grid(B * H, (S + kBQ - 1) / kBQ);
    hipLaunchKernelGGL((prefill_attention_kernel<DH>), grid, dim3(kThreads), 0, st, static_cast<const _Float16 *>(q),
                       static_cast<const _Float16 *>(kc), static_cast<const _Float16 *>(vc),
                       static_cast<_Float16 *>(ctx), static_cast<const _Float16 *>(alibi), pad, H, S, T_cap, scale,
                       pairs_per_group(64, (int)grid.y, B * H));
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
    // grid: (batch, head) pairs in x, query blocks in y
    EET_REQUIRE((long long)B * H < (1ll << 31) && (S + kBQ - 1) / kBQ <= 65535, EET_ERR_UNSUPPORTED_SHAPE,
                "eet_prefill_attention: B*H = %lld or S = %d too large", (long long)B * H, S);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dh) {
        case 32: return launch<32>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        case 64: return launch<64>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        case 96: return launch<96>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
        default: break;
    }
    // head size 128: the DMA kernel; it addresses a (b, h) cache range with 32-bit byte offsets and reads the
    // bias row in 4-byte units
    const bool alibi_ok = alibi == nullptr || (S % 2 == 0 && reinterpret_cast<uintptr_t>(alibi) % 4 == 0);
    if ((long long)S * 256 < (1ll << 31) && alibi_ok && eet::tuning().prefill_legacy == 0)
        return launch_dh128(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
    return launch<128>(q, k_cache, v_cache, ctx, alibi, pad, B, H, S, T_cap, st);
}
