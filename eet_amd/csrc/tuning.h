// Tuning overrides of the launch-shape tables, for sweeps and for the tests that
// run every kernel variant.  Nothing on the launch path reads the environment:
// the overrides live in one process-wide block that is written only by
// eet_set_tuning() and, once at library load, from the environment when
// EET_HIP_TUNING=1 is set.  An override that names a kernel variant that does not
// exist is ignored by the dispatcher (the table's choice runs instead).
#pragma once

namespace eet {

struct Tuning {
    // EET_GEMM_SMALL_M_CONFIG = "nt,waves,u[,ksplit]" (ksplit 2: the pair split, with nt = 2)
    bool has_small_m = false;
    int small_m_nt = 0, small_m_waves = 0, small_m_u = 0, small_m_ksplit = 1;
    // EET_GEMM_LARGE_M_TILE = "tm,tn[,ksplit]"
    bool has_large_m = false;
    int large_m_tm = 0, large_m_tn = 0, large_m_ksplit = 0;  // ksplit 0: not given
    // EET_MMHA_NSPLIT, EET_MMHA_THREADS, EET_MMHA_UNROLL (0: not given)
    int mmha_nsplit = 0, mmha_threads = 0, mmha_ring = 0;
    // EET_PREFILL_LEGACY = 1: head size 128 takes the register-staged prefill attention kernel
    int prefill_legacy = 0;
    int prefill_shape = 0;   // 1, 2: launch shape of the head-size-128 prefill attention kernel; 0 = by prompt length
    int prefill_group = 0;   // EET_PREFILL_GROUP: (batch, head) pairs per XCD group of the prefill attention order; -1: ungrouped
    // EET_CHAIN_SPIN_LIMIT: polls before a chained wait gives up (-1: the default, 65536; 0 gives up at once);
    // EET_CHAIN_SLEEP: s_sleep(8) repetitions between two polls (0: the default, 1)
    int chain_spin_limit = -1, chain_sleep = 0;
};

const Tuning &tuning();

}  // namespace eet
