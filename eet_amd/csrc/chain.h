// Chained launches: a kernel that is enqueued WITHOUT the queue's barrier between it and its
// predecessor (hipExtAnyOrderLaunch), requests its first weight batches right away -- they
// depend on nothing -- and only then waits, in the kernel, for the completion counter of the
// launch that produces its activations.  The launch boundary of two dependent kernels (about
// 1.6 us of idle GPU plus the ramp of the new kernel) overlaps the predecessor's tail instead.
//
// Protocol (all through agent-scope accesses, which the XCDs' L2 caches keep coherent):
//   producer  writes its outputs with sc1 (write-through) stores, waits for them (vmcnt 0),
//             and one lane adds 1 to shard (workgroup % 8) of its launch's counter;
//   consumer  wavefront 0 of every workgroup polls the eight shards (sc1 loads) until their
//             sum reaches the producer's cumulative workgroup count, the rest of the
//             workgroup waits at a barrier; activations and residual rows are then read
//             with sc1 loads (never from a stale L1 line).
// The wait is BOUNDED: after `spin_limit` polls the workgroup gives up, sets the device error
// word and goes on (its results are then undefined, but every kernel exits and signals); the
// host reads the word with eet_chain_status.  Counters live in a file-scope device array and
// only ever grow (32-bit wrap-around arithmetic), so nothing is cleared between launches.
#pragma once
#include <hip/hip_runtime.h>

namespace eet {

constexpr int kChainShards = 8;          // counter shards of a launch (one per XCD)
constexpr int kChainShardStride = 64;    // 32-bit words between shards: 256 bytes, two cache lines

struct ChainLink {
    const unsigned *wait;   // shards of the predecessor's counter; nullptr: nothing to wait for
    unsigned wait_target;   // cumulative workgroup count that means "predecessor complete"
    unsigned *signal;       // shards of this launch's counter; nullptr: not chained
    unsigned *error;        // device error word (set to 1 when a wait gives up)
    int spin_limit;         // polls before a wait gives up (0: gives up without polling)
    int sleep;              // s_sleep(8) repetitions between two polls
};

constexpr int kChainOff = 0, kChainFirst = 1, kChainNext = 2;

// Host side (chain.hip).  mode kChainFirst: the launch is an ordinary one (ordered behind all
// earlier work of the stream), it only signals.  kChainNext: the launch may be issued with
// hipExtAnyOrderLaunch (*any_order = true) and waits for the previous chained launch, which
// must have been made on the same stream of the same device.  `workgroups` is the grid size
// of the launch being prepared.
int chain_link(const char *who, int mode, unsigned workgroups, hipStream_t st, ChainLink *out, bool *any_order);

#if defined(__HIP_DEVICE_COMPILE__)
// Called by every lane of the workgroup, before the first read of anything a predecessor wrote.
__device__ __forceinline__ void chain_wait(const ChainLink &l)
{
    if (l.wait != nullptr) {   // uniform over the launch
        if (threadIdx.x < 64) {
            const int lane = threadIdx.x;
            bool ok = false;
            for (int budget = l.spin_limit; budget > 0; --budget) {
                unsigned v = 0;
                if (lane < kChainShards)
                    v = __hip_atomic_load(l.wait + lane * kChainShardStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v += __shfl_xor(v, 1, 64);
                v += __shfl_xor(v, 2, 64);
                v += __shfl_xor(v, 4, 64);
                v = __builtin_amdgcn_readfirstlane(v);
                if ((int)(v - l.wait_target) >= 0) {
                    ok = true;
                    break;
                }
                for (int i = 0; i < l.sleep; ++i)
                    __builtin_amdgcn_s_sleep(8);
            }
            if (!ok && lane == 0)
                __hip_atomic_store(l.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
    }
    asm volatile("" ::: "memory");
}

// Called by every lane of the workgroup after its last output store (sc1 stores).
__device__ __forceinline__ void chain_signal(const ChainLink &l)
{
    if (l.signal != nullptr) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_fetch_add(l.signal + (blockIdx.x % kChainShards) * kChainShardStride, 1u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    }
}
#endif

}  // namespace eet
