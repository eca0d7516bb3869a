// Host side of chained launches (see chain.h): the completion counters, the per-device
// bookkeeping that hands each launch its wait / signal words, and eet_chain_status.
#include "chain.h"

#include <mutex>

#include "common.h"
#include "tuning.h"

namespace {

constexpr int kSlots = 64;                                                  // launches before a counter is reused
constexpr int kSlotWords = eet::kChainShards * eet::kChainShardStride;      // 2 KiB per launch
constexpr int kErrorWord = kSlots * kSlotWords;                             // the device error word sits behind the counters

// Zero when the code object is loaded; counters only ever grow.
static __device__ __align__(256) unsigned chain_words[kSlots * kSlotWords + 64];

constexpr int kMaxDevices = 64;

struct DeviceChain {
    unsigned *words = nullptr;          // device address of chain_words on this GPU
    unsigned total[kSlots] = {};        // host mirror: workgroups ever signalled into a slot
    int last = -1;                      // slot of the previous chained launch (-1: none)
    hipStream_t last_stream = nullptr;
};

DeviceChain g_chain[kMaxDevices];
std::mutex g_mutex;

int device_chain(const char *who, DeviceChain **out)
{
    int dev = -1;
    EET_HIP_CHECK(hipGetDevice(&dev));
    EET_REQUIRE(dev >= 0 && dev < kMaxDevices, EET_ERR_HIP, "%s: device ordinal %d out of range", who, dev);
    DeviceChain &c = g_chain[dev];
    if (c.words == nullptr) {
        void *addr = nullptr;
        EET_HIP_CHECK(hipGetSymbolAddress(&addr, HIP_SYMBOL(chain_words)));
        EET_REQUIRE(addr != nullptr, EET_ERR_HIP, "%s: no device address for the chain counters", who);
        c.words = static_cast<unsigned *>(addr);
    }
    *out = &c;
    return EET_OK;
}

}  // namespace

int eet::chain_link(const char *who, int mode, unsigned workgroups, hipStream_t st, ChainLink *out, bool *any_order)
{
    *out = ChainLink{nullptr, 0u, nullptr, nullptr, 0, 0};
    *any_order = false;
    if (mode == kChainOff)
        return EET_OK;
    EET_REQUIRE(mode == kChainFirst || mode == kChainNext, EET_ERR_INVALID_ARGUMENT, "%s: unknown chain mode %d", who, mode);
    std::lock_guard<std::mutex> lock(g_mutex);
    DeviceChain *c = nullptr;
    if (int rc = device_chain(who, &c))
        return rc;
    if (mode == kChainNext) {
        EET_REQUIRE(c->last >= 0 && c->last_stream == st, EET_ERR_INVALID_ARGUMENT,
                    "%s: EET_CHAIN_NEXT needs a previous chained launch on the same stream of this device", who);
        // a launch without the queue barrier cannot be a node of a captured graph
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        EET_HIP_CHECK(hipStreamIsCapturing(st, &cap));
        EET_REQUIRE(cap == hipStreamCaptureStatusNone, EET_ERR_INVALID_ARGUMENT,
                    "%s: chained launches cannot be recorded into a HIP graph", who);
        out->wait = c->words + c->last * kSlotWords;
        out->wait_target = c->total[c->last];
        *any_order = true;
    }
    const int slot = (c->last + 1) % kSlots;
    c->total[slot] += workgroups;
    c->last = slot;
    c->last_stream = st;
    out->signal = c->words + slot * kSlotWords;
    out->error = c->words + kErrorWord;
    const eet::Tuning &t = eet::tuning();
    out->spin_limit = t.chain_spin_limit >= 0 ? t.chain_spin_limit : (1 << 16);
    out->sleep = t.chain_sleep > 0 ? t.chain_sleep : 1;
    return EET_OK;
}

extern "C" int eet_chain_status(int *gave_up, int clear, void *stream)
{
    EET_REQUIRE(gave_up != nullptr, EET_ERR_INVALID_ARGUMENT, "eet_chain_status: null pointer");
    std::lock_guard<std::mutex> lock(g_mutex);
    DeviceChain *c = nullptr;
    if (int rc = device_chain("eet_chain_status", &c))
        return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    EET_HIP_CHECK(hipStreamSynchronize(st));
    unsigned word = 0;
    EET_HIP_CHECK(hipMemcpy(&word, c->words + kErrorWord, sizeof(word), hipMemcpyDeviceToHost));
    if (clear && word != 0) {
        const unsigned zero = 0;
        EET_HIP_CHECK(hipMemcpy(c->words + kErrorWord, &zero, sizeof(zero), hipMemcpyHostToDevice));
    }
    *gave_up = word != 0 ? 1 : 0;
    return EET_OK;
}
