// Process-wide tuning overrides (see tuning.h) and the C entry point that sets them.
#include "tuning.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "common.h"

namespace {

eet::Tuning g_tuning;

int apply(const char *name, const char *value)
{
    eet::Tuning &t = g_tuning;
    const bool clear = value == nullptr || value[0] == '\0';
    if (std::strcmp(name, "EET_GEMM_SMALL_M_CONFIG") == 0) {
        t.has_small_m = false;
        if (clear)
            return EET_OK;
        t.small_m_ksplit = 1;
        if (std::sscanf(value, "%d,%d,%d,%d", &t.small_m_nt, &t.small_m_waves, &t.small_m_u, &t.small_m_ksplit) < 3)
            return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_set_tuning: %s wants \"nt,waves,u[,ksplit]\", got \"%s\"", name,
                             value);
        t.has_small_m = true;
        return EET_OK;
    }
    if (std::strcmp(name, "EET_GEMM_LARGE_M_TILE") == 0) {
        t.has_large_m = false;
        if (clear)
            return EET_OK;
        t.large_m_ksplit = 0;
        if (std::sscanf(value, "%d,%d,%d", &t.large_m_tm, &t.large_m_tn, &t.large_m_ksplit) < 2)
            return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_set_tuning: %s wants \"tm,tn[,ksplit]\", got \"%s\"", name,
                             value);
        t.has_large_m = true;
        return EET_OK;
    }
    int *slot = nullptr;
    if (std::strcmp(name, "EET_MMHA_NSPLIT") == 0)
        slot = &t.mmha_nsplit;
    else if (std::strcmp(name, "EET_MMHA_THREADS") == 0)
        slot = &t.mmha_threads;
    else if (std::strcmp(name, "EET_MMHA_UNROLL") == 0)
        slot = &t.mmha_ring;
    else if (std::strcmp(name, "EET_PREFILL_LEGACY") == 0)
        slot = &t.prefill_legacy;
    else if (std::strcmp(name, "EET_PREFILL_SHAPE") == 0)
        slot = &t.prefill_shape;
    else if (std::strcmp(name, "EET_PREFILL_GROUP") == 0)
        slot = &t.prefill_group;
    else if (std::strcmp(name, "EET_CHAIN_SLEEP") == 0)
        slot = &t.chain_sleep;
    else if (std::strcmp(name, "EET_CHAIN_SPIN_LIMIT") == 0) {
        t.chain_spin_limit = clear ? -1 : std::atoi(value);
        return EET_OK;
    }
    if (slot == nullptr)
        return eet::fail(EET_ERR_INVALID_ARGUMENT, "eet_set_tuning: unknown key \"%s\"", name);
    *slot = clear ? 0 : std::atoi(value);
    return EET_OK;
}

// once, when the library is loaded, and only on request
struct EnvInit {
    EnvInit()
    {
        const char *on = std::getenv("EET_HIP_TUNING");
        if (on == nullptr || std::strcmp(on, "1") != 0)
            return;
        for (const char *name : {"EET_GEMM_SMALL_M_CONFIG", "EET_GEMM_LARGE_M_TILE", "EET_MMHA_NSPLIT",
                                 "EET_MMHA_THREADS", "EET_MMHA_UNROLL", "EET_PREFILL_LEGACY", "EET_PREFILL_SHAPE", "EET_PREFILL_GROUP",
                                 "EET_CHAIN_SLEEP", "EET_CHAIN_SPIN_LIMIT"})
            if (const char *v = std::getenv(name))
                if (apply(name, v) != EET_OK)
                    std::fprintf(stderr, "[EET][WARN] %s\n", eet::last_error_slot().c_str());
    }
} g_env_init;

}  // namespace

const eet::Tuning &eet::tuning() { return g_tuning; }

extern "C" int eet_set_tuning(const char *name, const char *value)
{
    EET_REQUIRE(name != nullptr, EET_ERR_INVALID_ARGUMENT, "eet_set_tuning: null name");
    return apply(name, value);
}
