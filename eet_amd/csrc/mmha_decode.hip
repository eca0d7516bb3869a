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
// streams one contiguous range.  A workgroup of 512 lanes serves one (b, h):
// every group of dh/8 lanes streams its own rows with a running softmax and a
// small ring of rows in flight, and the streams meet once in LDS.  Only when
// there are fewer (b, h) pairs than CUs is the time axis split over `nsplit`
// workgroups (the reference runs one block per head); each then writes an
// un-normalised partial (max, sum, acc[dh]) and a second small kernel merges
// them.  There is no per-launch limit on step.
#if defined(EET_TIMELINE)
// Bench-only build of this file (linked into libeet_bench.so): the same kernels with clock readings per
// workgroup, under entry-point names of their own.
#define eet_rope_table eet_timeline_rope_table
#define eet_mmha_decode_workspace eet_timeline_mmha_decode_workspace
#define eet_mmha_decode eet_timeline_mmha_decode
#define eet_step_advance eet_timeline_step_advance
#define eet_mmha_decode_replayable_workspace eet_timeline_mmha_decode_replayable_workspace
#define eet_mmha_decode_replayable eet_timeline_mmha_decode_replayable
#define eet_mmha_decode_static_capacity eet_timeline_mmha_decode_static_capacity
#define eet_mmha_decode_static eet_timeline_mmha_decode_static
#endif
#include <hip/hip_runtime.h>

#include <cmath>

#include "common.h"
#include "tuning.h"

#if defined(EET_TIMELINE)
#define EET_ATL_PARAM , unsigned long long *tl
#define EET_ATL_ARG , attn_timeline_next((int)(grid.x * grid.y))
#define EET_ATL_STAMP(i)                                   \
    do {                                                   \
        if (tl != nullptr && threadIdx.x == 0)             \
            tl_t[i] = wall_clock64();                      \
    } while (0)
namespace {
constexpr int kAtlStamps = 8, kAtlMaxWgs = 2048;
unsigned long long *g_atl_buf = nullptr;   // [launch][kAtlMaxWgs][kAtlStamps], device memory
int g_atl_cap = 0, g_atl_n = 0;
int g_atl_grid[1024];
unsigned long long *attn_timeline_next(int workgroups)
{
    if (g_atl_buf == nullptr || g_atl_n >= g_atl_cap || g_atl_n >= 1024 || workgroups > kAtlMaxWgs)
        return nullptr;
    g_atl_grid[g_atl_n] = workgroups;
    return g_atl_buf + (size_t)(g_atl_n++) * kAtlMaxWgs * kAtlStamps;
}
}  // namespace
#else
#define EET_ATL_PARAM
#define EET_ATL_ARG
#define EET_ATL_STAMP(i)
#endif

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// A row of DH halves is DH/8 slices of 16 bytes, one per lane; the lanes of a row
// form a group of lanes_per_row(DH) (a power of two, so that the group sum is a
// butterfly): for DH = 96 four of the sixteen lanes of a group hold no slice, ask
// out of range (zeros, no memory touched) and add nothing.
constexpr int slices_per_row(int dh) { return dh / 8; }
constexpr int lanes_per_row(int dh) { return dh == 96 ? 16 : dh / 8; }

template <int WIDTH>
__device__ __forceinline__ float group_sum(float v)
{
#pragma unroll
    for (int off = WIDTH / 2; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

// NeoX rotary on one 8-element slice.  x holds elements d = 8*sub .. 8*sub+7 of
// a head row, y the slice DH/2 away; cs / sn are cos and sin of the position for
// the slice's 8 pairs (entries (sub % (DH/16)) * 8 .. of the table row
// [cos(DH/2) | sin(DH/2)]).  fp32 math, one rounding to fp16
// (csrc/core/common.cuh:209-225).
template <int DH>
__device__ __forceinline__ u32x4 rotate8(const u32x4 &x, const u32x4 &y, int sub, const float (&cs)[8],
                                         const float (&sn)[8])
{
    const bool lower = sub < slices_per_row(DH) / 2;
    const half8 hx = __builtin_bit_cast(half8, x), hy = __builtin_bit_cast(half8, y);
    half8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float a = (float)hx[e], b = (float)hy[e];
        o[e] = (_Float16)(lower ? a * cs[e] - b * sn[e] : a * cs[e] + b * sn[e]);
    }
    return __builtin_bit_cast(u32x4, o);
}

// DH: head size.  The DH/8 slices of a row are covered by one 16-byte load per lane.
// One query per (b, h) attends rows [0, step); grid = (B*H, nsplit).
template <int DH, int UN, int THREADS>
__global__ __launch_bounds__(THREADS) void mmha_decode_split_kernel(
    const _Float16 *__restrict__ q, const _Float16 *__restrict__ k_new, const _Float16 *__restrict__ v_new,
    long qkv_stride, _Float16 *__restrict__ k_cache, _Float16 *__restrict__ v_cache, _Float16 *__restrict__ ctx,
    const _Float16 *__restrict__ alibi, const int64_t *__restrict__ pad, float *__restrict__ partial, int H,
    int step, int T_cap, int nsplit, float scale, const float *__restrict__ rope_row,
    const int *__restrict__ step_dev, int alibi_ld_arg EET_ATL_PARAM)
{
#if defined(EET_TIMELINE)
    unsigned long long tl_t[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
    EET_ATL_STAMP(0);
    // Replayable form (a launch recorded into a HIP graph): the step lives in device
    // memory, rope_row is the base of the whole rotary table and the bias rows have a
    // fixed leading dimension, so that the same recorded arguments serve every step.
    // `step` arrives as step_max, the largest step the recording was sized for (launch
    // shape, rotary table rows, bias leading dimension): a step outside [1, step_max]
    // is clamped into it, so that no replay reads past those.
    if (step_dev != nullptr) {
        step = min(max(*step_dev, 1), min(step, T_cap));
        if (rope_row != nullptr)
            rope_row += (size_t)(step - 1) * DH;
    }
    constexpr int LPR = lanes_per_row(DH);   // lanes per row
    constexpr int NS = slices_per_row(DH);   // of which this many hold a slice
    constexpr int RPB = THREADS / LPR;       // row streams of the block (one per group of LPR lanes)
    __shared__ float accs[RPB][DH + 1];
    __shared__ float stream_m[RPB], stream_l[RPB], stream_w[RPB], merged_max;

    const int split = blockIdx.y;
    const int bh = blockIdx.x;
    const int alibi_ld = alibi_ld_arg > 0 ? alibi_ld_arg : step;
    const int b = bh / H, h = bh % H;
    const int tid = threadIdx.x;
    const int sub = tid % LPR;   // which 8-element slice of the row
    const int rs = tid / LPR;    // which row stream
    const bool holds = sub < NS;                         // false only for the idle lanes of DH = 96
    const unsigned idle = holds ? 0u : 0x80000000u;      // or-ed into buffer offsets: out of range
    const int pair = sub < NS / 2 ? sub + NS / 2 : sub - NS / 2;   // the slice DH/2 away (rotary partner)

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
    // (A sequence whose padding covers the new token too has no such row; split 0
    // appends it all the same, as the reference does, and gives it no weight.)
    const bool own_last = k_new != nullptr && step - 1 >= t0 && step - 1 < t1;
    const bool append = own_last || (k_new != nullptr && span == 0 && split == 0);
    // The requests for the new token's q, k, v and the rotary row go out first and
    // are consumed only after the first cache rows have been requested as well
    // (below), so the two memory latencies overlap.
    // They go through buffer resources of size zero when there is nothing to read
    // (no append, no rotary row): zeros come back and no branch surrounds the loads.
    const int r_last = own_last ? step - 1 - t0 : -1;
    u32x4 knew, kpair, vnew, qv;
    float rcs[8], rsn[8];
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    {
        const unsigned row_bytes = append ? (unsigned)(DH * 2) : 0u;
        const __amdgpu_buffer_rsrc_t knr = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<_Float16 *>(append ? k_new + qoff : q), 0, row_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t vnr = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<_Float16 *>(append ? v_new + qoff : q), 0, row_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t rpr = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float *>(rope_row ? rope_row : reinterpret_cast<const float *>(q)), 0,
            rope_row ? (unsigned)(DH * 4) : 0u, 0x00020000);
        const __amdgpu_buffer_rsrc_t qr = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(q + qoff), 0,
                                                                            (unsigned)(DH * 2), 0x00020000);
        const unsigned i0 = (unsigned)(sub % (NS / 2)) * 8u;
        knew = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(knr, (unsigned)sub * 16u | idle, 0, 0));
        kpair = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(knr, (unsigned)pair * 16u | idle, 0, 0));
        vnew = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(vnr, (unsigned)sub * 16u | idle, 0, 0));
        qv = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(qr, (unsigned)sub * 16u | idle, 0, 0));
        const u32x4 c0 = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rpr, i0 * 4u | idle, 0, 0));
        const u32x4 c1 = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rpr, (i0 * 4u + 16u) | idle, 0, 0));
        const u32x4 s0 =
            __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rpr, (DH / 2 + i0) * 4u | idle, 0, 0));
        const u32x4 s1 =
            __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rpr, ((DH / 2 + i0) * 4u + 16u) | idle, 0, 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            rcs[e] = __uint_as_float(c0[e]);
            rcs[4 + e] = __uint_as_float(c1[e]);
            rsn[e] = __uint_as_float(s0[e]);
            rsn[4 + e] = __uint_as_float(s1[e]);
        }
    }
#endif

    // Every group of LPR lanes walks its own stream of rows (rs, rs + RPB, ...)
    // with a running softmax (max m, sum l, un-normalised acc).  The K and V rows
    // (and the ALiBi term) of a stream sit in a ring of UN register slots: row i
    // is consumed from slot i % UN and the request for row i + UN goes out in its
    // place, so UN rows per stream stay in flight from the first row to the last
    // and nothing synchronises the workgroup until the streams are merged.
    // The cache range of this workgroup is addressed through buffer resources
    // whose size is exactly its n rows: requests past the end return zeros
    // without touching memory, which keeps the loop free of branches around loads.
#if defined(__HIP_DEVICE_COMPILE__)  // buffer-resource builtins exist in the device pass only
    const unsigned range_bytes = (unsigned)n * (unsigned)(DH * 2);
    const __amdgpu_buffer_rsrc_t krs =
        __builtin_amdgcn_make_buffer_rsrc(kc + (size_t)t0 * DH, 0, range_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs =
        __builtin_amdgcn_make_buffer_rsrc(vc + (size_t)t0 * DH, 0, range_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ars = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(alibi ? alibi + (size_t)h * alibi_ld + t0 : q), 0, alibi ? (unsigned)n * 2u : 0u,
        0x00020000);
    constexpr int kStream = 2;  // aux bits of a buffer load: non-temporal (every row is read exactly once)
    auto row_off = [&](int i) { return (unsigned)((rs + i * RPB) * (DH * 2) + sub * 16) | idle; };
    // Slot u is consumed first and refilled afterwards, so a slot's registers are
    // never live twice and the compiler keeps every slot in place: with the refill
    // ahead of the use it moved freshly requested registers at the end of each pass,
    // which waits for them and empties the ring.  The bias term sits in a 32-bit
    // register per slot (sign-extending load): pairs of 16-bit values get packed,
    // which is a move of a pending load again.
    u32x4 kv[UN], vv[UN];
    int ab[UN];
    auto request = [&](int u, int i) {
        kv[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(krs, row_off(i), 0, kStream));
        vv[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(vrs, row_off(i), 0, kStream));
        ab[u] = (int)(short)__builtin_amdgcn_raw_buffer_load_b16(ars, (unsigned)((rs + i * RPB) * 2), 0, 0);
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        request(u, u);
        __builtin_amdgcn_sched_barrier(0);
    }
    // Now the new token: rotate and append k, rotate q.  Their requests are older
    // than the ring's, so waiting for them leaves the ring in flight.
    {
        const u32x4 krot = rotate8<DH>(knew, kpair, sub, rcs, rsn);
        u32x4 qy;
        const int from = (int)(tid & 63) + pair - sub;   // the lane of this group that holds the partner slice
        qy.x = __shfl(qv.x, from, 64);
        qy.y = __shfl(qv.y, from, 64);
        qy.z = __shfl(qv.z, from, 64);
        qy.w = __shfl(qv.w, from, 64);
        const u32x4 qrot = rotate8<DH>(qv, qy, sub, rcs, rsn);
        if (rope_row != nullptr) {
            knew = krot;
            qv = qrot;
        }
        if (append && rs == 0 && holds) {
            *reinterpret_cast<u32x4 *>(kc + (size_t)(step - 1) * DH + sub * 8) = knew;
            *reinterpret_cast<u32x4 *>(vc + (size_t)(step - 1) * DH + sub * 8) = vnew;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    EET_ATL_STAMP(1);   // new token rotated and appended, the ring requested
    float m_run = -INFINITY, l_run = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int iters = (n + RPB - 1) / RPB;  // the same for every stream of the workgroup
    for (int i0 = 0; i0 < iters; i0 += UN) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int r = rs + (i0 + u) * RPB;  // the same for all LPR lanes of a group
            if (r < n) {   // uniform over the LPR lanes of a group, so the group sum below is whole
                u32x4 kcur = kv[u], vcur = vv[u];
                if (r == r_last) {  // the row being appended by this launch is still in registers
                    kcur = knew;
                    vcur = vnew;
                }
                float d = group_sum<LPR>(dot8(qv, kcur)) * scale;
                d += (float)__builtin_bit_cast(_Float16, (unsigned short)ab[u]);  // 0 without ALiBi
                const float m_new = fmaxf(m_run, d);
                const float c = __expf(m_run - m_new);  // 0 on the first row (m_run = -inf)
                const float p = __expf(d - m_new);
                l_run = l_run * c + p;
                const half8 hv = __builtin_bit_cast(half8, vcur);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    acc[e] = acc[e] * c + p * (float)hv[e];
                m_run = m_new;
            }
            __builtin_amdgcn_sched_barrier(0);
            request(u, i0 + u + UN);
            __builtin_amdgcn_sched_barrier(0);
#if defined(EET_TIMELINE)
            if (i0 == 0 && u == 0)
                EET_ATL_STAMP(2);   // the first row of this stream consumed
#endif
        }
    }
    EET_ATL_STAMP(3);   // the first wavefront's streams are through their rows
#else
    float m_run = -INFINITY, l_run = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#endif

    // Merge the RPB streams of the workgroup.
    if (holds) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            accs[rs][sub * 8 + e] = acc[e];
    }
    if (sub == 0) {
        stream_m[rs] = m_run;
        stream_l[rs] = l_run;
    }
    __syncthreads();
    EET_ATL_STAMP(4);   // every wavefront of the workgroup is through
    // The weight of every stream in the merge, exp(m - max over the streams), is computed once, by one lane per
    // stream, and the lanes that own an output element then only multiply and add (with the exponentials inside
    // their loop the merge took 1.3 us of a 24 us launch).
    if (tid < RPB) {
        float lmax = -INFINITY;
#pragma unroll 8
        for (int r = 0; r < RPB; ++r)
            lmax = fmaxf(lmax, stream_m[r]);
        const float mr = stream_m[tid];
        stream_w[tid] = (mr == -INFINITY) ? 0.f : __expf(mr - lmax);
        if (tid == 0)
            merged_max = lmax;
    }
    __syncthreads();
    if (tid < DH) {
        const float lmax = merged_max;
        float s = 0.f, lsum = 0.f;
#pragma unroll 8
        for (int r = 0; r < RPB; ++r) {
            const float w = stream_w[r];
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
#if defined(EET_TIMELINE)
    EET_ATL_STAMP(5);   // streams merged, result stores issued
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    EET_ATL_STAMP(6);   // ... and acknowledged
    if (tl != nullptr && threadIdx.x == 0) {
        unsigned long long *o = tl + (size_t)(blockIdx.y * gridDim.x + blockIdx.x) * kAtlStamps;
        for (int i = 0; i < 8; ++i)
            o[i] = tl_t[i];
    }
#endif
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

// How a launch is cut: `nsplit` workgroups of `threads` lanes per (b, h), each
// stream with a ring of `ring` rows.  Measured on MI355X (B*H = 256 at step ~1100
// and B*H = 1280 at step ~2200, 256 / 512 / 1024 lanes x 1..16 splits x rings of
// 2, 4, 8): 512 lanes (32 row streams at dh = 128) and no split is the fastest on
// both -- 25 us and 211 us, against 27-36 us and 217-224 us for the other widths --
// and shallow rings beat deep ones (more resident wavefronts matter more than
// more rows in flight per stream).  With fewer than 256 (b, h) pairs the time
// axis is split until there is one workgroup per CU, as long as a split keeps
// 256 rows; a short cache (under 8 rows per stream) takes 256-lane workgroups.
struct Plan {
    int threads, nsplit, ring;
};

Plan pick_plan(int BH, int dh, int step)
{
    const eet::Tuning &tune = eet::tuning();
    const int forced_ns = tune.mmha_nsplit, forced_threads = tune.mmha_threads, forced_ring = tune.mmha_ring;
    Plan p{512, 1, 4};
    const int want = (256 + BH - 1) / BH, by_rows = step / 256;
    p.nsplit = want < by_rows ? want : by_rows;
    if (p.nsplit < 1)
        p.nsplit = 1;
    if (forced_ns > 0)
        p.nsplit = forced_ns;
    if (forced_threads == 256 || forced_threads == 512 || forced_threads == 1024)
        p.threads = forced_threads;
    else if (step / p.nsplit / (p.threads / lanes_per_row(dh)) < 8)
        p.threads = 256;
    const int rows_per_stream = step / p.nsplit / (p.threads / lanes_per_row(dh));
    p.ring = rows_per_stream < 64 ? 2 : 4;
    if (forced_ring == 2 || forced_ring == 4 || forced_ring == 8)
        p.ring = forced_ring;
    return p;
}

template <int DH, int THREADS>
int launch_split(const void *q, const void *k, const void *v, long qkv_stride, void *kc, void *vc, void *ctx,
                 const void *alibi, const int64_t *pad, int B, int H, int step, int T_cap, void *ws, Plan plan,
                 const float *rope_row, hipStream_t st, const int *step_dev = nullptr, int alibi_ld = 0)
{
    const float scale = (float)(_Float16)(1.0f / sqrtf((float)DH));
    const int nsplit = plan.nsplit;
    dim3 grid(B * H, nsplit);
    auto kern = (plan.ring == 8)   ? mmha_decode_split_kernel<DH, 8, THREADS>
                : (plan.ring == 2) ? mmha_decode_split_kernel<DH, 2, THREADS>
                                   : mmha_decode_split_kernel<DH, 4, THREADS>;
    hipLaunchKernelGGL(kern, grid, dim3(THREADS), 0, st,
                       static_cast<const _Float16 *>(q), static_cast<const _Float16 *>(k),
                       static_cast<const _Float16 *>(v), qkv_stride, static_cast<_Float16 *>(kc),
                       static_cast<_Float16 *>(vc), static_cast<_Float16 *>(ctx),
                       static_cast<const _Float16 *>(alibi), pad, static_cast<float *>(ws), H, step, T_cap, nsplit,
                       scale, rope_row, step_dev, alibi_ld EET_ATL_ARG);
    EET_HIP_CHECK(hipGetLastError());
    if (nsplit > 1) {
        hipLaunchKernelGGL((mmha_decode_merge_kernel<DH>), dim3(B * H), dim3(DH), 0, st,
                           static_cast<const float *>(ws), static_cast<_Float16 *>(ctx), nsplit);
        EET_HIP_CHECK(hipGetLastError());
    }
    return EET_OK;
}

template <int DH>
int launch(const void *q, const void *k, const void *v, long qkv_stride, void *kc, void *vc, void *ctx,
           const void *alibi, const int64_t *pad, int B, int H, int step, int T_cap, void *ws, Plan plan,
           const float *rope_row, hipStream_t st, const int *step_dev = nullptr, int alibi_ld = 0)
{
    if (plan.threads == 1024)
        return launch_split<DH, 1024>(q, k, v, qkv_stride, kc, vc, ctx, alibi, pad, B, H, step, T_cap, ws, plan,
                                      rope_row, st, step_dev, alibi_ld);
    if (plan.threads == 512)
        return launch_split<DH, 512>(q, k, v, qkv_stride, kc, vc, ctx, alibi, pad, B, H, step, T_cap, ws, plan,
                                     rope_row, st, step_dev, alibi_ld);
    return launch_split<DH, 256>(q, k, v, qkv_stride, kc, vc, ctx, alibi, pad, B, H, step, T_cap, ws, plan, rope_row,
                                 st, step_dev, alibi_ld);
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
    const int ns = pick_plan(B * H, dh, step).nsplit;
    return ns > 1 ? (size_t)B * H * ns * (dh + 2) * sizeof(float) : 0;
}

// Argument checks shared by the two entry points; fills `plan`.
static int check_mmha_args(const char *fn, const void *q, const void *k, const void *v, long qkv_stride,
                           const void *k_cache, const void *v_cache, const void *ctx, int B, int H, int dh, int step,
                           int T_cap, const float *rope_cos_sin, Plan *plan)
{
    EET_REQUIRE(q && k_cache && v_cache && ctx, EET_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
    EET_REQUIRE((k == nullptr) == (v == nullptr), EET_ERR_INVALID_ARGUMENT,
                "%s: k and v must both be given or both be NULL", fn);
    EET_REQUIRE(B > 0 && H > 0 && step > 0 && T_cap > 0, EET_ERR_INVALID_ARGUMENT,
                "%s: bad sizes B=%d H=%d step=%d T_cap=%d", fn, B, H, step, T_cap);
    EET_REQUIRE(step <= T_cap, EET_ERR_INVALID_ARGUMENT, "%s: step %d exceeds the cache capacity %d", fn, step, T_cap);
    EET_REQUIRE(dh == 32 || dh == 64 || dh == 96 || dh == 128, EET_ERR_UNSUPPORTED_SHAPE,
                "%s: head size %d not supported (32, 64, 96, 128)", fn, dh);
    EET_REQUIRE(qkv_stride >= 0 && qkv_stride % 8 == 0, EET_ERR_INVALID_ARGUMENT,
                "%s: qkv_stride must be a non-negative multiple of 8", fn);
    EET_REQUIRE(rope_cos_sin == nullptr || k != nullptr, EET_ERR_INVALID_ARGUMENT,
                "%s: a rotary row needs the new k, v (it rotates q and the appended k)", fn);
    *plan = pick_plan(B * H, dh, step);
    return EET_OK;
}

static int run_mmha(const void *q, const void *k, const void *v, long qkv_stride, void *k_cache, void *v_cache,
                    void *ctx, const void *alibi, const int64_t *pad, int B, int H, int dh, int step, int T_cap,
                    const float *rope_cos_sin, void *partials, Plan plan, hipStream_t st,
                    const int *step_dev = nullptr, int alibi_ld = 0)
{
    switch (dh) {
        case 32:
            return launch<32>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, partials,
                              plan, rope_cos_sin, st, step_dev, alibi_ld);
        case 64:
            return launch<64>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, partials,
                              plan, rope_cos_sin, st, step_dev, alibi_ld);
        case 96:
            return launch<96>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, partials,
                              plan, rope_cos_sin, st, step_dev, alibi_ld);
        default:
            return launch<128>(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, step, T_cap, partials,
                               plan, rope_cos_sin, st, step_dev, alibi_ld);
    }
}

extern "C" int eet_mmha_decode(const void *q, const void *k, const void *v, long qkv_stride, void *k_cache,
                               void *v_cache, void *ctx, const void *alibi, const int64_t *pad, int B, int H,
                               int dh, int step, int T_cap, const float *rope_cos_sin, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    Plan plan;
    if (int rc = check_mmha_args("eet_mmha_decode", q, k, v, qkv_stride, k_cache, v_cache, ctx, B, H, dh, step,
                                 T_cap, rope_cos_sin, &plan))
        return rc;
    const size_t need = plan.nsplit > 1 ? (size_t)B * H * plan.nsplit * (dh + 2) * sizeof(float) : 0;
    EET_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), EET_ERR_WORKSPACE,
                "eet_mmha_decode: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return run_mmha(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, dh, step, T_cap, rope_cos_sin,
                    workspace, plan, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------
// Replayable form: the step comes from device memory, so the launch can be
// recorded once into a HIP graph and replayed for every token.
// ---------------------------------------------------------------------------
namespace {
__global__ void step_advance_kernel(int *step, int by) { *step += by; }
}  // namespace

extern "C" int eet_step_advance(int *step_dev, int by, void *stream)
{
    EET_REQUIRE(step_dev != nullptr, EET_ERR_INVALID_ARGUMENT, "eet_step_advance: null pointer");
    hipLaunchKernelGGL(step_advance_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), step_dev, by);
    EET_HIP_CHECK(hipGetLastError());
    return EET_OK;
}

extern "C" size_t eet_mmha_decode_replayable_workspace(int B, int H, int dh, int step_max)
{
    return eet_mmha_decode_workspace(B, H, dh, step_max);
}

extern "C" int eet_mmha_decode_replayable(const void *q, const void *k, const void *v, long qkv_stride, void *k_cache,
                                          void *v_cache, void *ctx, const void *alibi, int alibi_ld, const int64_t *pad,
                                          int B, int H, int dh, const int *step_dev, int step_max, int T_cap,
                                          const float *rope_table, void *workspace, size_t workspace_bytes,
                                          void *stream)
{
    EET_REQUIRE(step_dev != nullptr, EET_ERR_INVALID_ARGUMENT, "eet_mmha_decode_replayable: null step pointer");
    EET_REQUIRE(alibi == nullptr || alibi_ld >= step_max, EET_ERR_INVALID_ARGUMENT,
                "eet_mmha_decode_replayable: the bias rows need a leading dimension of at least step_max (%d), got %d",
                step_max, alibi_ld);
    Plan plan;
    if (int rc = check_mmha_args("eet_mmha_decode_replayable", q, k, v, qkv_stride, k_cache, v_cache, ctx, B, H, dh,
                                 step_max, T_cap, rope_table, &plan))
        return rc;
    const size_t need = plan.nsplit > 1 ? (size_t)B * H * plan.nsplit * (dh + 2) * sizeof(float) : 0;
    EET_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), EET_ERR_WORKSPACE,
                "eet_mmha_decode_replayable: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    // the launch shape is that of step_max; the kernel reads the step of each replay itself
    return run_mmha(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, dh, step_max, T_cap, rope_table,
                    workspace, plan, static_cast<hipStream_t>(stream), step_dev, alibi_ld);
}

// ---------------------------------------------------------------------------
// The same call for callers that cannot allocate: the split partials live in a
// file-scope device array instead of a caller-supplied workspace.
// ---------------------------------------------------------------------------
namespace {

// Largest split launch the static entry point takes: B*H*nsplit <= 512 partial
// records of (max, sum, acc[dh <= 128]) floats.  The table splits only when
// B*H < 256 and never into more than ceil(256 / (B*H)) parts, so every shape it
// chooses by itself fits (B*H*nsplit < 256 + B*H).
constexpr size_t kScratchRecords = 512;
constexpr size_t kScratchFloats = kScratchRecords * (128 + 2);

static __device__ __align__(256) float scratch[kScratchFloats];

// Device address of `scratch` per GPU (each device holds its own copy of the
// array at its own address); looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices];

int scratch_for_current_device(float **out)
{
    int dev = -1;
    EET_HIP_CHECK(hipGetDevice(&dev));
    EET_REQUIRE(dev >= 0 && dev < kMaxDevices, EET_ERR_HIP, "eet_mmha_decode_static: device ordinal %d out of range", dev);
    float *p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        void *addr = nullptr;
        EET_HIP_CHECK(hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)));
        EET_REQUIRE(addr != nullptr, EET_ERR_HIP, "eet_mmha_decode_static: no device address for the scratch array");
        p = static_cast<float *>(addr);
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);  // racing threads store the same address
    }
    *out = p;
    return EET_OK;
}

}  // namespace

extern "C" size_t eet_mmha_decode_static_capacity(void) { return kScratchFloats * sizeof(float); }

extern "C" int eet_mmha_decode_static(const void *q, const void *k, const void *v, long qkv_stride, void *k_cache,
                                      void *v_cache, void *ctx, const void *alibi, const int64_t *pad, int B, int H,
                                      int dh, int step, int T_cap, const float *rope_cos_sin, void *stream)
{
    Plan plan;
    if (int rc = check_mmha_args("eet_mmha_decode_static", q, k, v, qkv_stride, k_cache, v_cache, ctx, B, H, dh, step,
                                 T_cap, rope_cos_sin, &plan))
        return rc;
    const size_t need = plan.nsplit > 1 ? (size_t)B * H * plan.nsplit * (dh + 2) * sizeof(float) : 0;
    EET_REQUIRE(need <= kScratchFloats * sizeof(float), EET_ERR_WORKSPACE,
                "eet_mmha_decode_static: B*H*nsplit = %d*%d*%d partial records (%zu bytes) exceed the static scratch of "
                "%zu bytes; use eet_mmha_decode with a workspace",
                B, H, plan.nsplit, need, kScratchFloats * sizeof(float));
    float *partials = nullptr;
    if (int rc = scratch_for_current_device(&partials))
        return rc;
    // Every partial record a launch reads was written by the same launch's first
    // kernel, so nothing has to be cleared between calls.
    return run_mmha(q, k, v, qkv_stride, k_cache, v_cache, ctx, alibi, pad, B, H, dh, step, T_cap, rope_cos_sin,
                    partials, plan, static_cast<hipStream_t>(stream));
}

#if defined(EET_TIMELINE)
// Bench-only: recording starts with a device buffer for `launches` launches; every decode-attention launch made
// through the eet_timeline_mmha_* entry points from then on fills the next slot.  eet_timeline_attn_read
// synchronises the device, copies slot `launch` ([workgroup][8] readings of the 100 MHz wall clock: entry, ring
// requested, first row consumed, first wavefront through its rows, all wavefronts through, result stores issued,
// stores acknowledged) and returns the workgroup count of that launch, or a negative value.
extern "C" int eet_timeline_attn_begin(int launches)
{
    if (g_atl_buf != nullptr && g_atl_cap < launches) {
        (void)hipFree(g_atl_buf);
        g_atl_buf = nullptr;
    }
    if (g_atl_buf == nullptr) {
        EET_HIP_CHECK(hipMalloc(&g_atl_buf, (size_t)launches * kAtlMaxWgs * kAtlStamps * sizeof(unsigned long long)));
        g_atl_cap = launches;
    }
    EET_HIP_CHECK(hipMemset(g_atl_buf, 0, (size_t)g_atl_cap * kAtlMaxWgs * kAtlStamps * sizeof(unsigned long long)));
    g_atl_n = 0;
    return EET_OK;
}

extern "C" int eet_timeline_attn_read(int launch, unsigned long long *host_dst)
{
    if (launch < 0 || launch >= g_atl_n || host_dst == nullptr)
        return -1;
    if (hipDeviceSynchronize() != hipSuccess)
        return -2;
    const int wgs = g_atl_grid[launch];
    if (hipMemcpy(host_dst, g_atl_buf + (size_t)launch * kAtlMaxWgs * kAtlStamps,
                  (size_t)wgs * kAtlStamps * sizeof(unsigned long long), hipMemcpyDeviceToHost) != hipSuccess)
        return -2;
    return wgs;
}
#endif
